// C ABI of libjoshua_hip.so (declared in include/joshua_hip.h): weight objects
// resident in HBM in native GGUF block layout, shape validation with the
// reference's error behaviour, and kernel dispatch.
#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <map>
#include <tuple>
#include <memory>
#include <set>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/joshua_hip.h"
#include "kernels_mfma_q4k.hpp"
#include "kernels_graph.hpp"
#include "kernels_mla.hpp"
#include "kernels_mfma_q4k_gemm.hpp"
#include "kernels_mfma_q4k_stream.hpp"
#include "kernels_dot4_q4k.hpp"
#include "kernels_gemv_mfma.hpp"
#include "kernels_dot4_q6k.hpp"
#include "kernels_dot4_q8.hpp"
#include "kernels_moe.hpp"
#include "kernels_moe_mfma.hpp"
#include "kernels_gemv_mfma_tile.hpp"
#include "kernels_mfma_q4k_ring.hpp"
#include "kernels_moe_q4k_quads.hpp"
#include "kernels_mfma_q4k_rows16.hpp"
#include "kernels_mfma_q4k_gemm_i8.hpp"
#include "kernels_valu.hpp"
#include "kernels_mfma_decoded.hpp"

namespace {

thread_local char g_err[512] = "";
// Name of the kernel the calling thread's last matmul dispatch chose (jq_last_kernel).
thread_local const char *g_last_kernel = "";
void note_kernel(const char *name) { g_last_kernel = name; }

int fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return 1;
}

#define HIP_TRY(expr)                                                                      \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) return fail("%s: %s", #expr, hipGetErrorString(e_));         \
    } while (0)

struct Geometry {
    size_t elems, bytes;
};

bool geometry(uint32_t t, Geometry *g) {
    switch (t) {  // reference: src/gguf_ext.rs:483-512
    case JQ_TYPE_Q8_0: *g = {32, 34}; return true;
    case JQ_TYPE_Q2_K: *g = {256, 84}; return true;
    case JQ_TYPE_Q4_K: *g = {256, 144}; return true;
    case JQ_TYPE_Q6_K: *g = {256, 210}; return true;
    case JQ_TYPE_IQ2_XXS: *g = {256, 66}; return true;
    case JQ_TYPE_MXFP4: *g = {32, 17}; return true;
    case JQ_TYPE_Q4_0: *g = {32, 18}; return true;
    case JQ_TYPE_Q4_1: *g = {32, 20}; return true;
    case JQ_TYPE_Q5_0: *g = {32, 22}; return true;
    case JQ_TYPE_Q5_1: *g = {32, 24}; return true;
    case JQ_TYPE_Q3_K: *g = {256, 110}; return true;
    case JQ_TYPE_Q5_K: *g = {256, 176}; return true;
    default: return false;
    }
}

const char *type_name(uint32_t t) {
    switch (t) {
    case JQ_TYPE_Q8_0: return "quantized";
    case JQ_TYPE_Q2_K: return "quantized";
    case JQ_TYPE_Q4_K: return "quantized";
    case JQ_TYPE_Q6_K: return "quantized";
    case JQ_TYPE_Q4_0: case JQ_TYPE_Q4_1: case JQ_TYPE_Q5_0: case JQ_TYPE_Q5_1: case JQ_TYPE_Q3_K: case JQ_TYPE_Q5_K:
        return "quantized";
    case JQ_TYPE_IQ2_XXS: return "iq2_xxs";
    case JQ_TYPE_MXFP4: return "mxfp4";
    default: return "unknown";
    }
}

// Every block format the library decodes: X(type id, trait).
#define JQ_FOR_EACH_FORMAT(X) \
    X(JQ_TYPE_Q8_0, Q8_0) X(JQ_TYPE_Q2_K, Q2_K) X(JQ_TYPE_Q4_K, Q4_K) X(JQ_TYPE_Q6_K, Q6_K) X(JQ_TYPE_IQ2_XXS, IQ2_XXS) \
    X(JQ_TYPE_MXFP4, MXFP4) X(JQ_TYPE_Q4_0, Q4_0) X(JQ_TYPE_Q4_1, Q4_1) X(JQ_TYPE_Q5_0, Q5_0) X(JQ_TYPE_Q5_1, Q5_1)  \
    X(JQ_TYPE_Q3_K, Q3_K) X(JQ_TYPE_Q5_K, Q5_K)

std::once_flag g_init_once;
int g_init_rc = 0;
int g_device = 0;

}  // namespace

// Scratch memory of jq_matmul_t_noalloc: a fixed array in every device's memory, held from the moment the
// library is loaded on that device until the process ends.  Host code never uses the array's name as an
// address (on the host it is a stand-in, not device memory): noalloc_scratch_on() asks the runtime for the
// array's address on a device, once, with that device current, and every launch gets that pointer.
static __device__ __align__(256) uint8_t scratch[JQ_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int MAX_DEVICES = 64;
uint8_t *g_scratch_ptr[MAX_DEVICES] = {};
std::mutex g_scratch_mu[MAX_DEVICES];  // one call at a time enqueues launches that use a device's array
std::mutex g_scratch_table_mu;

// The address of `scratch` on `device`, which must be the current device.
int noalloc_scratch_on(int device, uint8_t **out) {
    if (device < 0 || device >= MAX_DEVICES) return fail("device %d is beyond the %d this library keeps scratch for", device, MAX_DEVICES);
    std::lock_guard<std::mutex> g(g_scratch_table_mu);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return fail("hipGetSymbolAddress returned no address for the scratch array on device %d", device);
        g_scratch_ptr[device] = (uint8_t *)p;
    }
    *out = g_scratch_ptr[device];
    return 0;
}

int do_init(int device) {
    int count = 0;
    HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return fail("jq_init: device %d out of range (%d visible)", device, count);
    HIP_TRY(hipSetDevice(device));
    g_device = device;
    uint8_t *p = nullptr;
    return noalloc_scratch_on(device, &p);
}

int ensure_init() {
    std::call_once(g_init_once, [] { g_init_rc = do_init(0); });
    return g_init_rc;
}

}  // namespace

struct jq_weight {
    uint32_t type;
    size_t n, k, nbytes, row_bytes;
    uint8_t *dev;
    bool owns;
};

namespace {

// Shape checks of the reference entry points, in their order and wording
// (reference: src/quant_matmul.rs:133-165, src/iq2xxs.rs:126-153,
// src/mxfp4.rs:142-172).
int validate(uint32_t type, size_t m, size_t k, size_t n, size_t lhs_len, size_t nbytes, size_t dst_len) {
    Geometry g;
    if (!geometry(type, &g)) return fail("unsupported tensor type id %u", type);
    if (k % g.elems != 0)
        return fail("%s matmul: k=%zu is not a multiple of the block size %zu", type_name(type), k, g.elems);
    size_t bpr = k / g.elems;
    if (nbytes % g.bytes != 0 || nbytes / g.bytes != n * bpr)
        return fail("%s matmul: rhs holds %zu blocks, expected %zu", type_name(type), nbytes / g.bytes, n * bpr);
    if (lhs_len != m * k || dst_len != m * n)
        return fail("%s matmul: lhs/dst sized %zu/%zu expected %zu/%zu", type_name(type), lhs_len, dst_len, m * k,
                    m * n);
    return 0;
}

template <class Q>
void launch_rows(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                 hipStream_t s) {
    dim3 grid((unsigned)((n + jq::ROWS_PER_WG - 1) / jq::ROWS_PER_WG)), block(64 * jq::ROWS_PER_WG);
    // rows staged through LDS when their starts are 16- or 4-byte aligned and four of them fit in 64 KB
    const size_t stride = (row_bytes + 15) / 16 * 16;
    const bool fits = stride * jq::ROWS_PER_WG + jq::table_bytes<Q>() <= 64 * 1024 && !getenv("JQ_NO_STAGED_ROWS");
    const int gran = !fits ? 0 : (row_bytes % 16 == 0 && ((uintptr_t)W & 15) == 0) ? 16
                                : (row_bytes % 4 == 0 && ((uintptr_t)W & 3) == 0)  ? 4 : 0;
    const size_t lds = stride * jq::ROWS_PER_WG + jq::table_bytes<Q>();
#define JQ_LAUNCH_ROWS(MT)                                                                                              \
    do {                                                                                                                 \
        if (gran == 16)                                                                                                  \
            hipLaunchKernelGGL((jq::matmul_rows_staged<Q, MT, 16>), grid, block, lds, s, W, row_bytes, X, Y, (int)m,     \
                               (int)k, (int)n, (int)stride);                                                             \
        else if (gran == 4)                                                                                              \
            hipLaunchKernelGGL((jq::matmul_rows_staged<Q, MT, 4>), grid, block, lds, s, W, row_bytes, X, Y, (int)m,      \
                               (int)k, (int)n, (int)stride);                                                             \
        else                                                                                                             \
            hipLaunchKernelGGL((jq::matmul_rows_valu<Q, MT>), grid, block, 0, s, W, row_bytes, X, Y, (int)m, (int)k,     \
                               (int)n);                                                                                  \
    } while (0)
    note_kernel(gran ? "matmul_rows_staged" : "matmul_rows_valu");
    if (m == 1) JQ_LAUNCH_ROWS(1);
    else if (m == 2) JQ_LAUNCH_ROWS(2);
    else JQ_LAUNCH_ROWS(4);
#undef JQ_LAUNCH_ROWS
}

// Q4_K, m <= 16: the MFMA decode kernel, up to four activation rows per launch.
constexpr size_t Q4K_MFMA_MAX_M = 16;
constexpr int LDS_LIMIT = 160 * 1024;

struct Q4kPlan {
    int units_per_tile, waves;
};

// Workgroup shape for a row length: all units of a tile in one workgroup, as
// many whole tiles as fit in 16 waves (JQ_Q4K_TILES_PER_WG overrides, for tuning).
bool q4k_plan(size_t k, size_t n, Q4kPlan *p) {
    int bpr = (int)(k / 256);
    int upt = (bpr + jq::Q4K_UNIT_BLOCKS - 1) / jq::Q4K_UNIT_BLOCKS;
    if (upt < 1 || upt > jq::Q4K_MAX_WAVES) return false;
    int tpw = std::max(1, 8 / upt);  // 8-wave workgroups measured best at 14336 x 4096
    static const int forced = [] {
        const char *e = getenv("JQ_Q4K_TILES_PER_WG");
        return e ? atoi(e) : 0;
    }();
    if (forced > 0 && forced * upt <= jq::Q4K_MAX_WAVES) tpw = forced;
    int tiles = (int)((n + 15) / 16);
    if (tpw > tiles) tpw = tiles;
    p->units_per_tile = upt;
    p->waves = tpw * upt;
    return true;
}

// Activation rows for the next launch: 4 when three or more are left (a
// fourth, absent row is masked), else what is left; fewer when LDS is short.
int q4k_mt_that_fits(size_t left, size_t k, int waves) {
    int first = left >= 3 ? 4 : (left == 2 ? 2 : 1);
    for (int mt = first; mt >= 1; mt >>= 1)
        if (jq::q4k_lds_layout((int)k, mt, waves).total <= LDS_LIMIT) return mt;
    return 0;
}

bool q4k_mfma_applies(size_t m, size_t k, size_t n) {
    Q4kPlan p;
    return m <= Q4K_MFMA_MAX_M && q4k_plan(k, n, &p) && jq::q4k_lds_layout((int)k, 1, p.waves).total <= LDS_LIMIT;
}

template <int MT>
int launch_q4k_mfma(const Q4kPlan &p, const uint8_t *W, size_t row_bytes, const float *X, float *Y, int m0, int m,
                    int k, int n, hipStream_t s) {
    static std::once_flag once;
    static hipError_t attr_rc = hipSuccess;
    std::call_once(once, [] {
        attr_rc = hipFuncSetAttribute((const void *)jq::q4k_gemv_mfma<MT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      LDS_LIMIT);
    });
    if (attr_rc != hipSuccess) return fail("hipFuncSetAttribute: %s", hipGetErrorString(attr_rc));
    int tiles = (n + 15) / 16, tpw = p.waves / p.units_per_tile;
    size_t lds = (size_t)jq::q4k_lds_layout(k, MT, p.waves).total;
    note_kernel("q4k_gemv_mfma");
    hipLaunchKernelGGL((jq::q4k_gemv_mfma<MT>), dim3((unsigned)((tiles + tpw - 1) / tpw)), dim3(64 * p.waves), lds, s, W,
                       row_bytes, X, Y, m0, m, k, n, p.units_per_tile);
    return 0;
}

int dispatch_q4k_mfma(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                      hipStream_t s) {
    Q4kPlan p;
    if (!q4k_plan(k, n, &p)) return fail("q4k mfma: unsupported row length %zu", k);
    for (size_t m0 = 0; m0 < m;) {
        int mt = q4k_mt_that_fits(m - m0, k, p.waves);
        int rc;
        switch (mt) {
        case 4: rc = launch_q4k_mfma<4>(p, W, row_bytes, X, Y, (int)m0, (int)m, (int)k, (int)n, s); break;
        case 2: rc = launch_q4k_mfma<2>(p, W, row_bytes, X, Y, (int)m0, (int)m, (int)k, (int)n, s); break;
        case 1: rc = launch_q4k_mfma<1>(p, W, row_bytes, X, Y, (int)m0, (int)m, (int)k, (int)n, s); break;
        default: return fail("q4k mfma: activations do not fit in LDS for k=%zu", k);
        }
        if (rc) return rc;
        m0 += (size_t)mt;
    }
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_K, one activation row: the integer-dot GEMVs.  By default the LDS-ring kernel takes rows of
// exactly 16 super-blocks (4096 wide: 10.15 us against 10.27 us for the MFMA GEMV on 14336 rows, and
// 2 % more decode tokens/s) and everything else is declined (-1).  JQ_Q4K_DOT4 = 0 turns them off,
// = regs selects the register-prefetch kernel for every row length up to 16 super-blocks.
// `norm`: residual add + RMSNorm in front of the product; `swiglu`: W pairs gate and up rows and Y gets
// the n / 2 activations (only the LDS-ring kernel has these forms).
int dispatch_q4k_dot4(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n, hipStream_t s,
                      const jq::QdNorm *norm = nullptr, bool swiglu = false) {
    const size_t nb = k / 256;
    static const char *mode_env = getenv("JQ_Q4K_DOT4");
    static const std::string mode = mode_env ? mode_env : "auto";
    if (mode == "0" || nb == 0 || row_bytes % 16 != 0 || ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0) return -1;
    // rows of 8 super-blocks (a 2048-wide hidden size), 64 weight rows or more: one workgroup of 8 waves a tile of 16
    // rows, with the decoder's norm form (4608 x 2048, q|k of a Qwen3-30B-A3B-shaped layer with residual add and RMSNorm:
    // one launch where there were rmsnorm_rows and the one-shot matrix-core GEMV).  JQ_Q4K_GEMV_TILE = 0 switches it off.
    static const char *tile_env = getenv("JQ_Q4K_GEMV_TILE");
    if (mode == "auto" && !swiglu && !(tile_env && tile_env[0] == '0') && nb == 8 && k == 2048 && row_bytes == nb * 144 &&
        n >= 64 && n <= 0x7FFFFFF0ull) {
        const jq::QdNorm nm = norm ? *norm : jq::QdNorm{};
        constexpr int lds = jq::gemv_mfma_tile_lds<jq::QvQ4K, 8>();
        static_assert(lds <= 64 * 1024, "within the default dynamic LDS limit");
        note_kernel("q4k_gemv_mfma_tile");
        if (norm)
            hipLaunchKernelGGL((jq::gemv_mfma_tile<jq::QvQ4K, 8, true>), dim3((unsigned)((n + 15) / 16)), dim3(512), lds, s, W, X, Y,
                               (int)n, nm.res, nm.w, nm.eps, nm.x_out, nm.hn_out);
        else
            hipLaunchKernelGGL((jq::gemv_mfma_tile<jq::QvQ4K, 8, false>), dim3((unsigned)((n + 15) / 16)), dim3(512), lds, s, W, X, Y,
                               (int)n, nullptr, nullptr, 0.0f, nullptr, nullptr);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    // rows of more than 16 super-blocks (up to 64: rows of 4352 to 16384 columns, contiguous), 512 weight rows or
    // more: the matrix-core kernel over two to four passes of 16 columns (4096 x 12288, a feed-forward down
    // projection: 7.2 us, where v_dot4 kernels in steps of 8 and 16 rows took 8.9; 4096 x 8192 5.6 against 6.5;
    // 7168 x 16384 15.7 us against 22.7 for the one-shot kernel).  JQ_Q4K_GEMV_COLS = 0 switches it off.
    static const char *cols_env = getenv("JQ_Q4K_GEMV_COLS");
    if (mode == "auto" && !norm && !swiglu && !(cols_env && cols_env[0] == '0') && nb > 16 && nb <= 64 &&
        row_bytes == nb * 144 && n >= 512 && n <= 0x7FFFFFF0ull) {
        const size_t tiles = (n + 15) / 16, rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
        const jq::QvColsWork wk{(int)n, (int)G, (int)(tiles / G), (int)(tiles % G), (int)nb};
        note_kernel("q4k_gemv_mfma_cols");
        if (nb <= 32) hipLaunchKernelGGL((jq::gemv_mfma_cols<jq::QvQ4K, 2>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, wk.nb);
        else if (nb <= 48) hipLaunchKernelGGL((jq::gemv_mfma_cols<jq::QvQ4K, 3>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, wk.nb);
        else hipLaunchKernelGGL((jq::gemv_mfma_cols<jq::QvQ4KCompact, 4>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, wk.nb);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    if (nb > jq::QD_MAX_WAVES) return -1;
    static const char *genv = getenv("JQ_Q4K_DOT4_GRID");
    const size_t tiles = (n + 15) / 16;
    if (mode != "regs") {
        if (nb != 16 || row_bytes != jq::QD_ROW) return -1;
        // from 2048 rows on, the product runs its dot products on the int8 matrix cores, with the norm and SwiGLU
        // forms of the decoder's fused launches (14336 rows: 7.1 against 7.9 us; 24576 rows with norm and SwiGLU:
        // 11.5 against 11.9; 4096: 3.8 against 4.3 us; a decoded token of the Qwen3-8B-shaped model 1.67 against
        // 1.74 ms)
        static const char *mfma_env = getenv("JQ_Q4K_GEMV_MFMA");
        static const size_t mfma_min_n = mfma_env ? (size_t)atoll(mfma_env) : 2048;
        if (!genv && mfma_min_n > 0 && n >= mfma_min_n && n <= 0x7FFFFFF0ull && (!swiglu || n % 2 == 0)) {
            const size_t rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
            const jq::QvWork wk{(int)n, (int)G, (int)(tiles / G), (int)(tiles % G)};
            const jq::QdNorm nm = norm ? *norm : jq::QdNorm{};
            note_kernel("q4k_gemv_mfma_lds");
#define JQ_MFMA_LDS(NORM, SWIGLU) \
    hipLaunchKernelGGL((jq::gemv_mfma_lds<jq::QvQ4K, NORM, SWIGLU>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, \
                       wk.rounds, wk.extra, nm.res, nm.w, nm.eps, nm.x_out, nm.hn_out)
            if (norm && swiglu) JQ_MFMA_LDS(true, true);
            else if (norm) JQ_MFMA_LDS(true, false);
            else if (swiglu) JQ_MFMA_LDS(false, true);
            else JQ_MFMA_LDS(false, false);
#undef JQ_MFMA_LDS
            HIP_TRY(hipGetLastError());
            return 0;
        }
        // a whole number of tiles per workgroup when the chip allows it (224 x 4 at 14336 rows)
        const size_t rounds = (tiles + 255) / 256;
        const unsigned grid = (unsigned)std::min<size_t>(tiles, genv ? (size_t)atoi(genv) : (tiles + rounds - 1) / rounds);
#define JQ_DOT4_LDS(NORM, SWIGLU, NM) \
    hipLaunchKernelGGL((jq::q4k_gemv_dot4_lds<NORM, SWIGLU>), dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid, \
                       NM.res, NM.w, NM.eps, NM.x_out, NM.hn_out)
        const jq::QdNorm none{};
        note_kernel("q4k_gemv_dot4_lds");
        if (norm && swiglu) JQ_DOT4_LDS(true, true, (*norm));
        else if (norm) JQ_DOT4_LDS(true, false, (*norm));
        else if (swiglu) JQ_DOT4_LDS(false, true, none);
        else JQ_DOT4_LDS(false, false, none);
#undef JQ_DOT4_LDS
        HIP_TRY(hipGetLastError());
        return 0;
    }
    if (norm || swiglu) return -1;
    // as many workgroups as the chip holds at once (one of 16 waves per CU, more when smaller), each
    // with an equal share of the rows
    const size_t cap = genv ? (size_t)atoi(genv) : 256 * std::max<size_t>(1, jq::QD_MAX_WAVES / nb);
    const unsigned grid = (unsigned)std::min<size_t>(tiles, std::max<size_t>(cap, 1));
    note_kernel("q4k_gemv_dot4");
    hipLaunchKernelGGL(jq::q4k_gemv_dot4, dim3(grid), dim3((unsigned)(64 * nb)), 0, s, W, row_bytes, X, Y, (int)k, (int)n);
    HIP_TRY(hipGetLastError());
    return 0;
}

// y1 = W1 hn and y2 = W2 hn in one launch, hn = rmsnorm(x + res) w: W1 Q4_K with 2048 rows or more of 4096 columns
// (the streaming kernel), W2 Q6_K or Q8_0 with few enough rows that G + n2 / 16 workgroups still run side by side.
// Returns -1 when the shapes are outside its reach.  JQ_NO_NORM_PAIR switches it off.
int dispatch_q4k_norm_pair(const uint8_t *W1, size_t row_bytes1, size_t n1, uint32_t type2, const uint8_t *W2, size_t row_bytes2,
                           size_t n2, size_t k, const float *X, float *Y1, float *Y2, const jq::QdNorm &nm, hipStream_t s) {
    static const char *off = getenv("JQ_NO_NORM_PAIR");
    static const char *dot4 = getenv("JQ_Q4K_DOT4"), *mfma = getenv("JQ_Q4K_GEMV_MFMA"), *no_norm = getenv("JQ_NO_FUSED_NORM");
    if (off || dot4 || mfma || no_norm || n2 == 0 || n2 % 16 != 0 || nm.hn_out || !nm.x_out || !nm.w) return -1;
    if ((((uintptr_t)W1 | (uintptr_t)W2 | (uintptr_t)X | (uintptr_t)nm.w | (uintptr_t)nm.res | (uintptr_t)nm.x_out) & 15) != 0) return -1;
    // rows of 2048 columns: both products a tile of 16 rows a workgroup of 8 waves
    static const char *tile_env = getenv("JQ_Q4K_GEMV_TILE");
    if (k == 2048 && row_bytes1 == 8 * 144 && n1 >= 64 && n1 <= 0x7FFFFFF0ull && !(tile_env && tile_env[0] == '0')) {
#define JQ_TPAIR(F2)                                                                                                       \
    do {                                                                                                                   \
        auto kern = jq::gemv_mfma_tile_norm_pair<jq::QvQ4K, F2, 8>;                                                        \
        constexpr int lds = jq::gemv_mfma_tile_pair_lds<jq::QvQ4K, F2, 8>();                                               \
        static const hipError_t attr_rc = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
        HIP_TRY(attr_rc);                                                                                                  \
        hipLaunchKernelGGL(kern, dim3((unsigned)((n1 + 15) / 16 + n2 / 16)), dim3(512), lds, s, W1, X, Y1, (int)n1, nm.res, nm.w, \
                           nm.eps, nm.x_out, W2, Y2, (int)n2);                                                             \
    } while (0)
        if (type2 == JQ_TYPE_Q6_K && row_bytes2 == 8 * 210) JQ_TPAIR(jq::QvQ6K);
        else if (type2 == JQ_TYPE_Q8_0 && row_bytes2 == 64 * 34) JQ_TPAIR(jq::QvI8<jq::Q8_0>);
        else return -1;
#undef JQ_TPAIR
        note_kernel("q4k_gemv_mfma_tile+pair");
        HIP_TRY(hipGetLastError());
        return 0;
    }
    if (k != 4096 || row_bytes1 != (size_t)jq::QvQ4K::ROW || n1 < 2048 || n1 > 0x7FFFFFF0ull) return -1;
    const size_t tiles = (n1 + 15) / 16, rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
    const size_t tiles2 = n2 / 16;
    if (G + tiles2 > 256) return -1;  // (one workgroup a compute unit: more would queue behind the streaming ones)
    const jq::QvWork wk{(int)n1, (int)G, (int)(tiles / G), (int)(tiles % G)};
#define JQ_PAIR(F2)                                                                                                        \
    do {                                                                                                                   \
        auto kern = jq::gemv_mfma_norm_pair<jq::QvQ4K, F2>;                                                                \
        constexpr int lds = jq::gemv_mfma_norm_pair_lds<jq::QvQ4K, F2>();                                                  \
        static_assert(lds <= 160 * 1024, "one workgroup's LDS");                                                          \
        static const hipError_t attr_rc = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds); \
        HIP_TRY(attr_rc);                                                                                                  \
        hipLaunchKernelGGL(kern, dim3((unsigned)(G + tiles2)), dim3(1024), lds, s, W1, X, Y1, wk.n, wk.G, wk.rounds, wk.extra, \
                           nm.res, nm.w, nm.eps, nm.x_out, W2, Y2, (int)n2);                                               \
    } while (0)
    if (type2 == JQ_TYPE_Q6_K && row_bytes2 == 16 * 210) JQ_PAIR(jq::QvQ6K);
    else if (type2 == JQ_TYPE_Q8_0 && row_bytes2 == 128 * 34) JQ_PAIR(jq::QvI8<jq::Q8_0>);
    else return -1;
#undef JQ_PAIR
    note_kernel("q4k_gemv_mfma_lds+pair");
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q2_K, one activation row, rows of 4096: the int8 matrix-core GEMV.  Returns -1 when the shape is outside
// its reach.  JQ_Q2K_GEMV_MFMA = 0 switches it off.
int dispatch_q2k_mfma(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n, hipStream_t s) {
    static const char *mode = getenv("JQ_Q2K_GEMV_MFMA");
    if ((mode && mode[0] == '0') || k != 4096 || row_bytes != (size_t)jq::QvQ2K::ROW || ((uintptr_t)W & 15) != 0 ||
        ((uintptr_t)X & 15) != 0 || n < 256 || n > 0x7FFFFFF0ull)
        return -1;
    const size_t tiles = (n + 15) / 16, rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
    const jq::QvWork wk{(int)n, (int)G, (int)(tiles / G), (int)(tiles % G)};
    note_kernel("q2k_gemv_mfma_lds");
    hipLaunchKernelGGL(jq::gemv_mfma_lds<jq::QvQ2K>, dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, nullptr, nullptr, 0.0f, nullptr, nullptr);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_0, Q4_1, Q5_0, Q5_1, Q5_K and Q3_K, one activation row, rows of 4096: the int8 matrix-core GEMV over the policy of
// the formats whose units decode to int8 codes with a scale and an offset (Q3_K: two scales a unit, signed codes).  Returns -1 when the shape is outside its
// reach (then the f32 row kernel runs).
template <class F>
int launch_i8_gemv(const char *name, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n,
                   hipStream_t s) {
    static const char *off = getenv("JQ_NO_I8_GEMV");
    if (off || k != 4096 || row_bytes != (size_t)F::ROW || ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0 || n < 256 ||
        n > 0x7FFFFFF0ull)
        return -1;
    const size_t tiles = (n + 15) / 16, rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
    const jq::QvWork wk{(int)n, (int)G, (int)(tiles / G), (int)(tiles % G)};
    note_kernel(name);
    hipLaunchKernelGGL(jq::gemv_mfma_lds<F>, dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, nullptr,
                       nullptr, 0.0f, nullptr, nullptr);
    HIP_TRY(hipGetLastError());
    return 0;
}

int dispatch_i8_gemv(uint32_t type, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n,
                     hipStream_t s) {
    switch (type) {
    case JQ_TYPE_Q4_0: return launch_i8_gemv<jq::QvI8<jq::Q4_0>>("q4_0_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    case JQ_TYPE_Q4_1: return launch_i8_gemv<jq::QvI8<jq::Q4_1>>("q4_1_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    case JQ_TYPE_Q5_0: return launch_i8_gemv<jq::QvI8<jq::Q5_0>>("q5_0_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    case JQ_TYPE_Q5_1: return launch_i8_gemv<jq::QvI8<jq::Q5_1>>("q5_1_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    case JQ_TYPE_Q5_K: return launch_i8_gemv<jq::QvI8<jq::Q5_K>>("q5k_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    case JQ_TYPE_Q3_K: return launch_i8_gemv<jq::QvQ3K>("q3k_gemv_mfma_lds", W, row_bytes, X, Y, k, n, s);
    default: return -1;
    }
}

// Q6_K, Q8_0 and Q5_K, one activation row, rows of 2048 columns, 64 weight rows or more: a tile of 16 rows a workgroup of
// 8 waves on the int8 matrix cores (the output head of a 2048-wide model, 151936 rows of Q6_K).  Returns -1 when the
// shape is outside its reach (then the f32 row kernel runs).
template <class F>
int launch_gemv_tile8(const char *name, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t n, hipStream_t s) {
    if (row_bytes != (size_t)8 * F::BLOCK) return -1;
    auto kern = jq::gemv_mfma_tile<F, 8, false>;
    constexpr int lds = jq::gemv_mfma_tile_lds<F, 8>();
    static const hipError_t attr_rc = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    HIP_TRY(attr_rc);
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3((unsigned)((n + 15) / 16)), dim3(512), lds, s, W, X, Y, (int)n, nullptr, nullptr, 0.0f, nullptr,
                       nullptr);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q8_0 and Q6_K, one activation row, rows of 4096 columns, at most 256 tiles of 16 weight rows (4096 x 4096: one tile a
// compute unit): the same kernel with 16 waves a tile, every byte of the matrix asked for at once.  JQ_GEMV_TILE16 = 0
// switches it off.
template <class F>
int launch_gemv_tile16(const char *name, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t n, hipStream_t s) {
    if (row_bytes != (size_t)16 * F::BLOCK) return -1;
    auto kern = jq::gemv_mfma_tile<F, 16, false>;
    constexpr int lds = jq::gemv_mfma_tile_lds<F, 16>();
    static_assert(lds <= 160 * 1024, "one workgroup's LDS");
    static const hipError_t attr_rc = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
    HIP_TRY(attr_rc);
    note_kernel(name);
    hipLaunchKernelGGL(kern, dim3((unsigned)((n + 15) / 16)), dim3(1024), lds, s, W, X, Y, (int)n, nullptr, nullptr, 0.0f, nullptr,
                       nullptr);
    HIP_TRY(hipGetLastError());
    return 0;
}

int dispatch_gemv_tile16(uint32_t type, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n,
                         hipStream_t s) {
    static const char *off = getenv("JQ_GEMV_TILE16");
    if ((off && off[0] == '0') || k != 4096 || n < 256 || n > 4096 || (((uintptr_t)W | (uintptr_t)X) & 15) != 0 ||
        row_bytes % 16 != 0)
        return -1;
    // (4096 x 4096: Q8_0 5.4 us against 5.7 on the v_dot4 kernel, Q6_K 5.6 against 6.2; 2048 rows of Q8_0 4.4 against 6.9 on
    // the f32 row kernel; Q6_K below 2048 rows stays on the f32 row kernel, 3.9 against 4.2 at 1024)
    switch (type) {
    case JQ_TYPE_Q6_K: return n < 2048 ? -1 : launch_gemv_tile16<jq::QvQ6K>("q6k_gemv_mfma_tile", W, row_bytes, X, Y, n, s);
    case JQ_TYPE_Q8_0: return launch_gemv_tile16<jq::QvI8<jq::Q8_0>>("q8_0_gemv_mfma_tile", W, row_bytes, X, Y, n, s);
    default: return -1;
    }
}

int dispatch_gemv_tile8(uint32_t type, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n,
                        hipStream_t s) {
    static const char *off = getenv("JQ_Q4K_GEMV_TILE");
    if ((off && off[0] == '0') || k != 2048 || n < 64 || n > 0x7FFFFFF0ull || (((uintptr_t)W | (uintptr_t)X) & 15) != 0 ||
        row_bytes % 16 != 0)
        return -1;
    switch (type) {
    case JQ_TYPE_Q6_K: return launch_gemv_tile8<jq::QvQ6K>("q6k_gemv_mfma_tile", W, row_bytes, X, Y, n, s);
    case JQ_TYPE_Q8_0: return launch_gemv_tile8<jq::QvI8<jq::Q8_0>>("q8_0_gemv_mfma_tile", W, row_bytes, X, Y, n, s);
    case JQ_TYPE_Q5_K: return launch_gemv_tile8<jq::QvI8<jq::Q5_K>>("q5k_gemv_mfma_tile", W, row_bytes, X, Y, n, s);
    default: return -1;
    }
}

// Q6_K, one activation row, rows of 4096, 8192 or 12288: the v_dot4 LDS-ring kernel.
// Returns -1 when the shape is outside its reach.
int dispatch_q6k_dot4(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n, hipStream_t s) {
    static const char *mode = getenv("JQ_Q6K_DOT4");
    const size_t ng = k / 4096;
    if ((mode && mode[0] == '0') || k % 4096 != 0 || ng < 1 || ng > 3 || row_bytes != ng * jq::Q6D_SLICE ||
        ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0)
        return -1;
    // The int8 matrix-core GEMV over the Q6_K policy, for rows of 8192 and 12288 columns and up to 8192 weight
    // rows (4096 x 12288, a feed-forward down projection: 11.4 us against 12.0 on v_dot4).  A tile of 16 rows is
    // 54 KB, so its ring has two slots and one tile in flight while a tile is multiplied: with more tiles a
    // workgroup, and at rows of 4096, the v_dot4 kernel's ring of three 8-row steps streams faster (151936 x 4096:
    // 87 against 92 us; 4096 x 4096: 6.1 us either way).  JQ_Q6K_GEMV_MFMA = 0 switches it off, = all takes
    // every shape it can.
    static const char *mfma_env = getenv("JQ_Q6K_GEMV_MFMA");
    const bool mfma_all = mfma_env && !strcmp(mfma_env, "all"), mfma_off = mfma_env && mfma_env[0] == '0';
    if (!mfma_off && n >= 256 && n <= 0x7FFFFFF0ull && (mfma_all || (ng >= 2 && n <= 8192))) {
        const size_t tiles16 = (n + 15) / 16, rounds_up = (tiles16 + 255) / 256, G = (tiles16 + rounds_up - 1) / rounds_up;
        const jq::QvColsWork wk{(int)n, (int)G, (int)(tiles16 / G), (int)(tiles16 % G), (int)(16 * ng)};
        note_kernel(ng == 1 ? "q6k_gemv_mfma_lds" : "q6k_gemv_mfma_cols");
        if (ng == 1)
            hipLaunchKernelGGL(jq::gemv_mfma_lds<jq::QvQ6K>, dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra,
                               nullptr, nullptr, 0.0f, nullptr, nullptr);
        else if (ng == 2)
            hipLaunchKernelGGL((jq::gemv_mfma_cols<jq::QvQ6K, 2>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, wk.nb);
        else
            hipLaunchKernelGGL((jq::gemv_mfma_cols<jq::QvQ6K, 3>), dim3((unsigned)G), dim3(1024), 0, s, W, X, Y, wk.n, wk.G, wk.rounds, wk.extra, wk.nb);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    const size_t tiles = (n + jq::Q6D_ROWS - 1) / jq::Q6D_ROWS, rounds = (tiles + 255) / 256;
    if (tiles * ng < 512) return -1;  // under two steps a workgroup the staged f32 kernel is as fast (5.9 vs 4.5 us at 1024 x 4096)
    static const char *genv = getenv("JQ_Q6K_DOT4_GRID");
    const unsigned grid = (unsigned)std::min<size_t>(tiles, genv ? (size_t)std::max(atoi(genv), 1) : (tiles + rounds - 1) / rounds);
    note_kernel("q6k_gemv_dot4_lds");
    if (ng == 1) hipLaunchKernelGGL(jq::q6k_gemv_dot4_lds<1>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    else if (ng == 2) hipLaunchKernelGGL(jq::q6k_gemv_dot4_lds<2>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    else hipLaunchKernelGGL(jq::q6k_gemv_dot4_lds<3>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q8_0, one activation row, rows of 4096, 8192 or 12288: the v_dot4 LDS-ring kernel.
// Returns -1 when the shape is outside its reach.
int dispatch_q8_0_dot4(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t k, size_t n, hipStream_t s) {
    static const char *mode = getenv("JQ_Q8_0_DOT4");
    const size_t ng = k / 4096;
    if ((mode && mode[0] == '0') || k % 4096 != 0 || ng < 1 || ng > 3 || row_bytes != ng * jq::Q8D_SLICE ||
        ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0)
        return -1;
    const size_t tiles = (n + jq::Q8D_ROWS - 1) / jq::Q8D_ROWS, rounds = (tiles + 255) / 256;
    if (tiles * ng < 512) return -1;  // under two steps a workgroup the staged f32 kernel is as fast
    const unsigned grid = (unsigned)std::min<size_t>(tiles, (tiles + rounds - 1) / rounds);
    note_kernel("q8_0_gemv_dot4_lds");
    if (ng == 1) hipLaunchKernelGGL(jq::q8_0_gemv_dot4_lds<1>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    else if (ng == 2) hipLaunchKernelGGL(jq::q8_0_gemv_dot4_lds<2>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    else hipLaunchKernelGGL(jq::q8_0_gemv_dot4_lds<3>, dim3(grid), dim3(1024), 0, s, W, X, Y, (int)n, (int)grid);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_K, 1..16 activation rows, rows of at most 16 super-blocks: the weight-streaming MFMA kernel.
// Returns -1 when the shape is outside its reach.
int dispatch_q4k_stream(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                        hipStream_t s) {
    const size_t nb = k / 256;
    static const char *off = getenv("JQ_Q4K_NO_STREAM");
    if (off || m > 16 || nb == 0 || nb > 16 || (nb > 8 && nb % 2 != 0) || row_bytes % 16 != 0 ||
        ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0)
        return -1;
    const int cpw = nb > 8 ? 2 : 1, waves = (int)(nb / cpw);
    const size_t n_tiles = (n + 15) / 16;
    static const char *genv = getenv("JQ_Q4K_STREAM_GRID");
    const size_t cap = genv ? (size_t)atoi(genv) : (cpw == 2 ? 256 : 512);
    const unsigned grid = (unsigned)std::min<size_t>(n_tiles, std::max<size_t>(cap, 1));
    note_kernel("q4k_stream_mfma");
    if (cpw == 2)
        hipLaunchKernelGGL(jq::q4k_stream_mfma<2>, dim3(grid), dim3(64 * waves), 0, s, W, row_bytes, X, Y, (int)m, (int)k, (int)n);
    else
        hipLaunchKernelGGL(jq::q4k_stream_mfma<1>, dim3(grid), dim3(64 * waves), 0, s, W, row_bytes, X, Y, (int)m, (int)k, (int)n);
    HIP_TRY(hipGetLastError());
    return 0;
}

// rows x k activations -> one MFMA operand record per (row, 256-element column)
void launch_q4k_acts_prep(const float *X, size_t rows, size_t k, uint8_t *out, hipStream_t s) {
    const size_t units = rows * (k / 256);
    hipLaunchKernelGGL(jq::q4k_acts_prep, dim3((unsigned)((units + 7) / 8)), dim3(256), 0, s, X, (int)rows, (int)k, out);
}

// Device memory for what one call's launches hand to each other (prepared activation operands, partial
// sums of a product split over k), on stream s.  Requests up to SCRATCH_KEEP bytes are served from one
// allocation per (device, stream), made at first use and kept until the process ends: the launches of a
// stream run in order, so consecutive calls can share it, and a call pays no allocator round trip
// (hipMallocAsync with hipFreeAsync takes some 18 us of host time a call, more than the kernels of a
// small matmul take on the device).  A call that needs more than the stream's buffer holds gets a new,
// larger one; the old one is retired, not freed, because a HIP graph captured earlier on the stream
// still names it (sizes at least double, so a stream retires at most a handful of buffers).  The holder
// keeps that allocation's lock until it goes out of scope, after the call's last launch is enqueued, so
// host threads that share a stream enqueue their calls one after the other.  Larger requests are
// stream-ordered allocations, freed behind the call's launches.  First use and growth allocate: neither
// is possible while the stream is being captured, so a caller warms a stream up with its largest call
// before capturing it.
//
// jq_matmul_t_noalloc serves the same requests from a fixed array in device memory instead (below): it
// installs the array for the calling thread with FixedScratchScope, and get() then hands out that
// array, or fails when the request exceeds it, and never reaches an allocator.
constexpr size_t SCRATCH_KEEP = 64u << 20;

struct StreamBuffer {
    std::mutex mu;
    uint8_t *ptr = nullptr;
    size_t bytes = 0;
    std::vector<uint8_t *> retired;
};

std::mutex g_stream_table_mu;
// keyed by (device, stream, kind): kind 0 is what a product's launches hand to each other, kind 1 the f32 copies of
// jq_matmul_t_f16's operands around such a product (which takes buffer 0 itself)
std::map<std::tuple<int, hipStream_t, int>, std::unique_ptr<StreamBuffer>> g_stream_table;

// jq_stream_release: waits for the stream, then frees its buffer and the retired ones.
int release_stream_scratch(hipStream_t s) {
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    std::vector<std::unique_ptr<StreamBuffer>> bufs;
    {
        std::lock_guard<std::mutex> g(g_stream_table_mu);
        for (int kind = 0; kind < 2; kind++) {
            auto it = g_stream_table.find({dev, s, kind});
            if (it == g_stream_table.end()) continue;
            bufs.push_back(std::move(it->second));
            g_stream_table.erase(it);
        }
    }
    if (bufs.empty()) return 0;
    for (auto &b : bufs) { std::lock_guard<std::mutex> wait_for_the_last_holder(b->mu); }
    HIP_TRY(hipStreamSynchronize(s));
    for (auto &b : bufs) {
        if (b->ptr) (void)hipFree(b->ptr);
        for (uint8_t *p : b->retired) (void)hipFree(p);
    }
    return 0;
}

struct FixedScratch {
    uint8_t *ptr = nullptr;
    size_t bytes = 0;
    std::mutex *mu = nullptr;
};
thread_local const FixedScratch *tl_fixed_scratch = nullptr;

struct FixedScratchScope {
    explicit FixedScratchScope(const FixedScratch *f) { tl_fixed_scratch = f; }
    ~FixedScratchScope() { tl_fixed_scratch = nullptr; }
};

class CallScratch {
    std::unique_lock<std::mutex> lock_;
    hipStream_t stream_ = nullptr;
    uint8_t *transient_ = nullptr;
    int kind_ = 0;

public:
    CallScratch() = default;
    explicit CallScratch(int kind) : kind_(kind) {}
    CallScratch(const CallScratch &) = delete;
    CallScratch &operator=(const CallScratch &) = delete;
    ~CallScratch() {
        if (transient_) (void)hipFreeAsync(transient_, stream_);
    }
    // 0 on success; on failure the message is set
    int get(size_t bytes, hipStream_t s, uint8_t **out) {
        stream_ = s;
        if (const FixedScratch *f = kind_ == 0 ? tl_fixed_scratch : nullptr) {
            if (bytes > f->bytes)
                return fail("this product needs %zu bytes of scratch memory; the entry point that allocates nothing "
                            "holds %zu", bytes, f->bytes);
            lock_ = std::unique_lock<std::mutex>(*f->mu);
            *out = f->ptr;
            return 0;
        }
        if (bytes > SCRATCH_KEEP) {
            HIP_TRY(hipMallocAsync((void **)&transient_, bytes, s));
            *out = transient_;
            return 0;
        }
        int dev = 0;
        HIP_TRY(hipGetDevice(&dev));
        StreamBuffer *b;
        {
            std::lock_guard<std::mutex> g(g_stream_table_mu);
            auto &slot = g_stream_table[{dev, s, kind_}];
            if (!slot) slot.reset(new StreamBuffer);
            b = slot.get();
        }
        lock_ = std::unique_lock<std::mutex>(b->mu);
        if (b->bytes < bytes) {
            const size_t want = std::min(SCRATCH_KEEP, std::max<size_t>({(bytes + 0xFFFFF) & ~(size_t)0xFFFFF, 2 * b->bytes,
                                                                          (size_t)1 << 20}));
            uint8_t *fresh = nullptr;
            HIP_TRY(hipMalloc((void **)&fresh, want));
            if (b->ptr) b->retired.push_back(b->ptr);
            b->ptr = fresh, b->bytes = want;
        }
        *out = b->ptr;
        return 0;
    }
};

// Workgroups of the LDS-ring MFMA kernel that fit a compute unit (LDS and the 16 waves of a SIMD group).
constexpr int ring_wgs_per_cu(int maxnb) { return maxnb == 16 ? 1 : maxnb == 8 ? 2 : 4; }

// Q4_K, 1..16 activation rows, contiguous rows of at most 16 super-blocks: the LDS-ring MFMA kernel.
// Returns -1 when the shape is outside its reach.
int dispatch_q4k_ring(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                      hipStream_t s) {
    const size_t nb = k / 256;
    static const char *off = getenv("JQ_Q4K_NO_RING");
    if (off || m > 16 || nb == 0 || nb > 16 || row_bytes != nb * 144 || ((uintptr_t)W & 15) != 0 ||
        ((uintptr_t)X & 15) != 0 || n > 0x7FFFFFF0ull)
        return -1;
    const int maxnb = nb > 8 ? 16 : nb > 4 ? 8 : 4;
    const size_t tiles = (n + 15) / 16, slots = 256 * (size_t)ring_wgs_per_cu(maxnb);
    static const char *genv = getenv("JQ_Q4K_RING_GRID");
    const size_t per = (tiles + slots - 1) / slots;
    const unsigned grid = genv ? (unsigned)std::max(atoi(genv), 1) : (unsigned)((tiles + per - 1) / per);
    // the activations as MFMA operand records, in the call scratch of the stream
    CallScratch scratch;
    uint8_t *acts = nullptr;
    if (scratch.get(m * nb * jq::QS_REC, s, &acts)) return 1;
    launch_q4k_acts_prep(X, m, k, acts, s);
#define JQ_RING(MAXNB)                                                                                              \
    hipLaunchKernelGGL((jq::q4k_ring_mfma<MAXNB, false, false>), dim3(grid), dim3(64 * (unsigned)nb), 0, s, W, nullptr, \
                       nullptr, acts, nullptr, nullptr, nullptr, nullptr, Y, (int)m, (int)n, jq::MoeClamp{})
    note_kernel("q4k_ring_mfma");
    if (maxnb == 16) JQ_RING(16);
    else if (maxnb == 8) JQ_RING(8);
    else JQ_RING(4);
#undef JQ_RING
    HIP_TRY(hipGetLastError());
    return 0;
}

// How many runs of super-blocks a GEMM of `total` workgroup tiles splits its k dimension into.  One tile
// list fills the 256 compute units only from 256 tiles on; a list of 32 tiles split eight ways does, at the
// price of writing and re-reading the partial sums.  Estimated per candidate from the measured step time of
// a workgroup (us per super-block, plus its start and end) and ~3 TB/s for the partial sums; the choice
// depends on the shape only, so a shape always gets the same order of additions.
// `other_bytes`: what the call keeps in its scratch beside the partial sums; with a scratch of fixed size (the
// entry point that allocates nothing) a split count whose partial sums would not fit is passed over.
int gemm_k_splits(size_t total, size_t nb, size_t m, size_t n, double us_per_block, const char *env,
                  double *estimate_us = nullptr, size_t other_bytes = 0) {
    if (env && !estimate_us) return (int)std::min<size_t>(std::max(atoi(env), 1), nb);
    const size_t cap = tl_fixed_scratch && !estimate_us ? tl_fixed_scratch->bytes : (size_t)1 << 60;
    int best = 1;
    double best_us = 0.0;
    for (size_t sp = 1; sp <= std::min<size_t>(nb, 16); sp++) {
        if (sp > 1 && other_bytes + sp * m * n * sizeof(float) > cap) continue;
        const double rounds = (double)((total * sp + 255) / 256);
        const double wg_us = 3.0 + us_per_block * (double)((nb + sp - 1) / sp);
        const double sum_us = sp == 1 ? 0.0 : 3.0 + (double)(2 * sp + 1) * (double)(m * n) * 4.0 / 3.0e6;
        const double us = rounds * wg_us + sum_us;
        if (sp == 1 || us < best_us * 0.95) best = (int)sp, best_us = us;
    }
    if (estimate_us) *estimate_us = best_us;
    return best;
}

// Estimated time of the Q4_K MFMA GEMM (dispatch_q4k_gemm) on an m x k by n x k product, in us.
double q4k_gemm_estimate_us(size_t m, size_t k, size_t n) {
    const size_t m_tiles = (m + jq::QG_MT - 1) / jq::QG_MT, n_tiles = (n + jq::QG_NT - 1) / jq::QG_NT;
    double us = 0.0;
    gemm_k_splits(m_tiles * n_tiles, k / 256, m, n, 6.0, nullptr, &us);
    return us;
}

// Q4_K, two activation rows or more, rows of 4096, 8192, 12288 or 16384 columns: the int8 matrix-core kernel
// on the one-row GEMV's weight stream, once per group of 16 activation rows and of 4096 columns (a matrix
// of this size stays in the last-level cache between the passes; later column groups add to the result), its operands prepared by one small launch into the call
// scratch of the stream.  Beyond 16 rows it runs while its estimated time (a pass costs ~4.3 us plus
// 0.53 us per 1024 weight rows) stays below the MFMA GEMM's.  Returns -1 when the shape is outside its reach.
constexpr size_t Q4K_ROWS16_MAX_M = 256;

int dispatch_q4k_rows16(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                        hipStream_t s) {
    static const char *off = getenv("JQ_Q4K_NO_ROWS16");
    static const char *min_env = getenv("JQ_Q4K_ROWS16_MIN_N");
    static const size_t min_n = min_env ? (size_t)atoll(min_env) : 1024;
    static const char *max_env = getenv("JQ_Q4K_ROWS16_MAX_M");
    static const size_t max_m = max_env ? std::min<size_t>((size_t)atoll(max_env), 1024) : Q4K_ROWS16_MAX_M;
    if (off || m < 2 || m > max_m || k == 0 || k % 4096 != 0 || k > 4 * 4096 || row_bytes % 16 != 0 ||
        row_bytes < k / 256 * 144 || n < min_n || n > 0x7FFFFFF0ull || ((uintptr_t)W & 15) != 0 || ((uintptr_t)X & 15) != 0)
        return -1;
    const size_t tiles = (n + 15) / 16, rounds = (tiles + 255) / 256, groups = (m + 15) / 16, col_groups = k / 4096;
    // a pass = 16 activation rows x 4096 columns over all weight rows
    const double passes_us = 3.0 + (double)(groups * col_groups) * (4.3 + 0.527 * (double)n / 1024.0);
    if ((groups > 1 || col_groups > 1) && !max_env && passes_us >= q4k_gemm_estimate_us(m, k, n)) return -1;
    if (col_groups > 1 && m < 3) return -1;  // two rows: the two-row GEMV walks the matrix once
    static const char *genv = getenv("JQ_Q4K_ROWS16_GRID");
    const unsigned grid = (unsigned)std::min<size_t>(tiles, genv ? (size_t)std::max(atoi(genv), 1) : (tiles + rounds - 1) / rounds);
    // rows of 4096 columns, one after the other: the streaming form of the kernel (JQ_Q4K_ROWS16_LDS = 0: the form before
    // it; = own: the activations quantised by every workgroup for itself instead of by the preparation launch, which
    // measured slower: every workgroup then reads all 16 rows of activations, 57 MB through the L2 for 224 workgroups)
    static const char *lds_env = getenv("JQ_Q4K_ROWS16_LDS");
    const bool lds_form = col_groups == 1 && row_bytes == (size_t)jq::QD_ROW && !genv && !(lds_env && lds_env[0] == '0');
    const size_t rounds_up = (tiles + 255) / 256, G = (tiles + rounds_up - 1) / rounds_up;
    if (lds_form && lds_env && !strcmp(lds_env, "own")) {
        note_kernel("q4k_rows16_lds");
        for (size_t g = 0; g < groups; g++)
            hipLaunchKernelGGL(jq::q4k_rows16_lds<true>, dim3((unsigned)G), dim3(1024), 0, s, W, X + 16 * g * k, nullptr,
                               Y + 16 * g * n, (int)std::min<size_t>(16, m - 16 * g), (int)n, (int)G, (int)(tiles / G),
                               (int)(tiles % G), (int)k);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    CallScratch scratch;
    uint8_t *acts = nullptr;
    const size_t cols = k / 256, group_bytes = cols * (size_t)jq::QM_REC;
    if (scratch.get(groups * group_bytes, s, &acts)) return 1;
    hipLaunchKernelGGL(jq::q4k_acts16_prep, dim3(8, (unsigned)cols, (unsigned)groups), dim3(64), 0, s, X, (int)m, (int)k, acts);
    if (lds_form) {
        note_kernel("q4k_rows16_lds");
        for (size_t g = 0; g < groups; g++)
            hipLaunchKernelGGL(jq::q4k_rows16_lds<false>, dim3((unsigned)G), dim3(1024), 0, s, W, X, (const uint8_t *)(acts + g * group_bytes),
                               Y + 16 * g * n, (int)std::min<size_t>(16, m - 16 * g), (int)n, (int)G, (int)(tiles / G),
                               (int)(tiles % G), (int)k);
        HIP_TRY(hipGetLastError());
        return 0;
    }
    note_kernel("q4k_rows16_mfma");
    for (size_t g = 0; g < groups; g++)
        for (size_t cg = 0; cg < col_groups; cg++)
            hipLaunchKernelGGL(jq::q4k_rows16_mfma, dim3(grid), dim3(1024), 0, s, W + cg * (size_t)jq::QD_ROW,
                               (const uint8_t *)(acts + g * group_bytes + 16 * cg * (size_t)jq::QM_REC), Y + 16 * g * n,
                               (int)std::min<size_t>(16, m - 16 * g), (int)n, (int)grid, row_bytes, (int)(cg > 0));
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_K, Q6_K, Q2_K and Q8_0 with many activation rows on the int8 matrix cores: the activations as two int8 planes per
// 256-element super-block in the call scratch of the stream, then kq_gemm_i8 with the workgroup shape and the
// split over k that an estimate fitted to measurements prefers.  Returns -1 when the shape is outside its
// reach or the product is tiny.  JQ_Q4K_GEMM_I8 = 0 switches it off; JQ_Q4K_GEMM_I8_SHAPE and _SPLITS force the
// choice, _MIN_TILES moves the floor (small tiles times the splits that k allows; default 64), _MIN_M the
// fewest activation rows (default: min_m_default, 64 for Q4_K, which has kernels of its own below that).
struct GemmI8Shape {
    int nw, ng;
    bool nsplit;  // tiles of 32 activation rows whose waves share the weight rows
};

template <class F>
int dispatch_gemm_i8(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                     hipStream_t s, const char *name, const char *name_split, bool swiglu_pairs = false,
                     size_t min_m_default = 64) {
    constexpr size_t ALIGN = F::ALIGN;
    static const char *mode = getenv("JQ_Q4K_GEMM_I8");
    static const char *min_tiles_env = getenv("JQ_Q4K_GEMM_I8_MIN_TILES");
    static const char *shape_env = getenv("JQ_Q4K_GEMM_I8_SHAPE");  // "waves,groups": one of the shapes below
    static const size_t min_tiles = min_tiles_env ? (size_t)atoll(min_tiles_env) : 64;
    // One activation scale per 256 elements resolves a row relative to its super-blocks' largest magnitudes:
    // that is the contract from 64 rows on (prefill); fewer rows keep the kernels with a scale per 32.
    static const char *min_m_env = getenv("JQ_Q4K_GEMM_I8_MIN_M");
    const size_t min_m = min_m_env ? std::max<size_t>((size_t)atoll(min_m_env), 2) : min_m_default;
    // fewer than 64 rows (the formats without a kernel of their own for them): against 8M weights or more; below
    // that the GEMM over decoded weights is as fast or faster (32 x 2048 x 2048: 16 us against 22)
    if (!min_m_env && m < 64 && n * k < ((size_t)8 << 20)) return -1;
    if ((mode && mode[0] == '0') || m < min_m || k % 256 != 0 || row_bytes % ALIGN != 0 || ((uintptr_t)W & (ALIGN - 1)) != 0 ||
        ((uintptr_t)X & 15) != 0 || m > 0x7FFFFFF0ull || n > 0x7FFFFFF0ull)
        return -1;
    // Two workgroup shapes: 256 x 112 outputs (eight waves, one workgroup a compute unit) and 128 x 64 (four
    // waves, two a compute unit), and a split over k (the parts summed by splitk_sum) when the tiles alone leave
    // compute units idle: every workgroup then walks nb / splits super-blocks.
    // Up to 32 rows also: 32 x 64 (two waves that share the weight rows, two workgroups a compute unit).
    static const GemmI8Shape shapes[] = {{8, 7, false}, {8, 6, false}, {4, 4, false}, {2, 4, true}};
    const size_t nb = k / 256, groups = (m + 15) / 16;
    auto tiles_of = [&](const GemmI8Shape &sh) {
        const size_t mt = sh.nsplit ? 32 : 32 * (size_t)sh.nw, nt = 16 * (size_t)sh.ng;
        return ((m + mt - 1) / mt) * ((n + nt - 1) / nt);
    };
    if (tiles_of(shapes[2]) * std::max<size_t>(1, std::min<size_t>(nb / 4, 8)) < min_tiles) return -1;
    // Estimate per (shape, splits), in us, fitted to whole-call times of Q4_K products of 32 to 2048 rows
    // against 1024 to 24576 weight rows of 4096 and 12288 columns (the picks are within 5 % of the best
    // measured choice there; Q6_K runs ~10 % longer with the same ordering): the preparation, a fixed part,
    // the super-blocks a workgroup walks at a cost that grows with the workgroups at work (a large workgroup:
    // 5.0 us a super-block with 74 at work, 6.6 with 256; a small one: 2.5 with 64, 3.0 with 256, 4.7 when two
    // share every compute unit), and the sum's launch and its (splits + 1) m n floats, which the last-level
    // cache holds.
    const size_t acts_bytes = (groups * nb * (size_t)jq::QI_REC + 255) & ~(size_t)255;
    const size_t scratch_cap = tl_fixed_scratch ? tl_fixed_scratch->bytes : (size_t)1 << 40;
    auto estimate = [&](const GemmI8Shape &sh, size_t sp) {
        const double wgs = (double)(tiles_of(sh) * sp), nbl = (double)(nb / sp);
        double us = 3.0 + 0.0035 * (double)(nb * groups);
        if (sh.nsplit)  // 3.1 us a super-block with 64 at work, 3.4 with 256, 4.4 with 512 (two a compute unit), in whole rounds
            us += 3.9 + nbl * (2.95 + 0.0029 * std::min(wgs, 512.0)) *
                            (wgs <= 512.0 ? 1.0 : wgs < 2048.0 ? std::ceil(wgs / 512.0) : wgs / 512.0);
        else if (sh.nw == 8)  // (six groups of weight rows instead of seven: six sevenths of the work a super-block)
            us += 10.0 + nbl * (4.3 + 0.009 * std::min(wgs, 256.0)) * std::ceil(wgs / 256.0) * (sh.ng == 7 ? 1.0 : 0.88);
        else if (wgs <= 256.0) us += 3.9 + nbl * (2.3 + 0.0027 * wgs);
        else us += 3.9 + nbl * (3.1 + 0.0032 * std::min(wgs, 512.0)) * std::max(1.0, wgs / 512.0);
        if (sp > 1) us += 1.0 + 0.8 * (double)sp + (double)(sp + 1) * (double)(m * n) * 4.0 / 8.0e6;
        return us;
    };
    const GemmI8Shape *best = nullptr;
    size_t splits = 1;
    double best_us = 0.0;
    static const char *splits_env = getenv("JQ_Q4K_GEMM_I8_SPLITS");
    int want_nw = 0, want_ng = 0;
    const bool forced = shape_env && sscanf(shape_env, "%d,%d", &want_nw, &want_ng) == 2;
    for (const GemmI8Shape &sh : shapes) {
        if (forced && (sh.nw != want_nw || sh.ng != want_ng)) continue;
        if (sh.nsplit && !forced && m > 32) continue;
        for (size_t sp = 1; sp <= 8; sp++) {
            if (nb % sp != 0 || (sp > 1 && nb / sp < 4)) continue;
            if (splits_env && sp != (size_t)atoi(splits_env)) continue;
            if (sp > 1 && (m * n > 0x3FFFFFFFull || acts_bytes + sp * m * n * sizeof(float) > scratch_cap)) continue;
            const double us = estimate(sh, sp);
            if (!best || us < best_us) best = &sh, splits = sp, best_us = us;
        }
    }
    if (!best) return -1;
    CallScratch scratch;
    uint8_t *acts = nullptr;
    if (scratch.get(acts_bytes + (splits > 1 ? splits * m * n * sizeof(float) : 0), s, &acts)) return 1;
    float *parts = (float *)(acts + acts_bytes);
    const size_t mt = best->nsplit ? 32 : 32 * (size_t)best->nw, nt = 16 * (size_t)best->ng;
    const size_t tx = (n + nt - 1) / nt, ty = (m + mt - 1) / mt;
    const size_t grid = 8 % ty == 0 ? (tx * ty + 7) / 8 * 8 : tx * ty;
    if (grid > 0x7FFFFFFFull) return -1;
    hipError_t attr_rc = hipSuccess;
#define JQ_GEMM_I8(NW_, NG_, NSPLIT_)                                                                                 \
    if (best->nw == NW_ && best->ng == NG_) {                                                                         \
        auto kern = jq::kq_gemm_i8<F, NW_, NG_, false, NSPLIT_>;                                                      \
        constexpr int lds = jq::qi_lds_bytes<F, NG_>();                                                                  \
        static std::once_flag big_lds;                                                                                \
        static hipError_t rc_once = hipSuccess;                                                                       \
        std::call_once(big_lds, [&] {                                                                                 \
            rc_once = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);       \
        });                                                                                                           \
        attr_rc = rc_once;                                                                                            \
        if (attr_rc == hipSuccess) {                                                                                  \
            if (swiglu_pairs)                                                                                         \
                hipLaunchKernelGGL((jq::q4k_gemm_i8_prep<true, F::SUB16>), dim3((unsigned)nb, (unsigned)groups), dim3(256), 0, s, \
                                   X, (int)m, (int)k, acts);                                                          \
            else                                                                                                      \
                hipLaunchKernelGGL((jq::q4k_gemm_i8_prep<false, F::SUB16>), dim3((unsigned)nb, (unsigned)groups), dim3(256), 0, s, \
                                   X, (int)m, (int)k, acts);                                                          \
            hipLaunchKernelGGL(kern, dim3((unsigned)grid, (unsigned)splits), dim3(64 * NW_), lds, s, W, row_bytes,    \
                               (const uint8_t *)acts, splits > 1 ? parts : Y, (int)m, (int)n, (int)(nb / splits),     \
                               (int)groups, (int)tx, (int)ty, (int)nb, splits > 1 ? m * n : (size_t)0, jq::QiGrouped{}); \
            if (splits > 1)                                                                                           \
                hipLaunchKernelGGL(jq::splitk_sum, dim3((unsigned)((m * n + 1023) / 1024)), dim3(256), 0, s, parts, Y, \
                                   m * n, (int)splits);                                                               \
        }                                                                                                             \
    }
    JQ_GEMM_I8(8, 7, false)
    JQ_GEMM_I8(8, 6, false)
    JQ_GEMM_I8(4, 4, false)
    JQ_GEMM_I8(2, 4, true)
#undef JQ_GEMM_I8
    if (attr_rc != hipSuccess) return fail("hipFuncSetAttribute: %s", hipGetErrorString(attr_rc));
    note_kernel(splits > 1 ? name_split : name);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_K with more than 16 activation rows: prepare the fixed-point activation planes in the
// call scratch of the stream, then the MFMA GEMM, split over k when its tiles alone would leave
// compute units idle.
int dispatch_q4k_gemm(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                      hipStream_t s) {
    constexpr size_t MT = jq::QG_MT;
    const size_t m_pad = (m + MT - 1) / MT * MT, nb = k / 256;
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t plane_bytes = up(m_pad * k * 2 * sizeof(uint16_t)), min_bytes = up(m_pad * nb * 64);
    const size_t m_tiles = m_pad / MT, n_tiles = (n + jq::QG_NT - 1) / jq::QG_NT, total = m_tiles * n_tiles;
    // 8 XCDs x the longest per-XCD work list (see the tile order at the top of the kernel)
    size_t per_xcd;
    if (m_tiles >= 8) per_xcd = (m_tiles + 7) / 8 * n_tiles;
    else if (8 % m_tiles != 0) per_xcd = (total + 7) / 8;
    else per_xcd = (n_tiles + 8 / m_tiles - 1) / (8 / m_tiles);
    const size_t base_grid = 8 * per_xcd;
    static const char *split_env = getenv("JQ_Q4K_GEMM_SPLITS");
    const size_t splits = m * n / 1024 < 0x7FFFFFFFull ? (size_t)gemm_k_splits(total, nb, m, n, 6.0, split_env, nullptr, plane_bytes + min_bytes) : 1;
    if (base_grid * splits > 0x0FFFFFFFull) return fail("q4k gemm: %zu x %zu tiles exceed the grid limit", m_tiles, n_tiles);
    const size_t part_bytes = splits > 1 ? splits * m * n * sizeof(float) : 0;
    CallScratch scratch;
    uint8_t *buf = nullptr;
    if (scratch.get(plane_bytes + min_bytes + part_bytes, s, &buf)) return 1;
    jq::Q4kGemmActs a;
    a.planes = (_Float16 *)buf;
    a.mins = (_Float16 *)(buf + plane_bytes);
    float *parts = (float *)(buf + plane_bytes + min_bytes);
    const size_t units = m_pad * nb;
    note_kernel(splits > 1 ? "q4k_gemm_mfma+splitk" : "q4k_gemm_mfma");
    hipLaunchKernelGGL(jq::q4k_gemm_prep, dim3((unsigned)((units + 3) / 4)), dim3(256), 0, s, X, (int)m, (int)m_pad, (int)k, a);
    hipLaunchKernelGGL(jq::q4k_gemm_mfma, dim3((unsigned)(base_grid * splits)), dim3(512), 0, s, W, row_bytes, a,
                       splits > 1 ? parts : Y, (int)m, (int)m_pad, (int)k, (int)n, (int)m_tiles, (int)total, (int)splits,
                       (int)base_grid, splits > 1 ? m * n : (size_t)0);
    if (splits > 1)
        hipLaunchKernelGGL(jq::splitk_sum, dim3((unsigned)((m * n + 1023) / 1024)), dim3(256), 0, s, parts, Y, m * n, (int)splits);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail("q4k gemm launch: %s", hipGetErrorString(e));
    return 0;
}

// Any format, more than 16 activation rows, k a multiple of 256: activations as two f16 planes in the
// call scratch of the stream, then the MFMA GEMM over decoded weights.  Returns -1 when the
// shape is outside its reach.
template <class Q>
int launch_gemm_decoded(const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m, size_t k, size_t n,
                        hipStream_t s) {
    static const char *off = getenv("JQ_NO_DECODED_GEMM");
    if (off || k % jq::GD_KC != 0 || ((uintptr_t)X & 15) != 0) return -1;
    const size_t m_pad = (m + jq::GD_MT - 1) / jq::GD_MT * jq::GD_MT, nc = k / jq::GD_KC;
    auto up = [](size_t v) { return (v + 255) / 256 * 256; };
    const size_t plane = up(m_pad * k * sizeof(_Float16)), sbytes = up(m_pad * nc * sizeof(float));
    // split over k when the 64 x 64 tiles alone leave compute units idle (a workgroup takes ~5 us a chunk)
    const size_t n_tiles = (n + jq::GD_NT - 1) / jq::GD_NT, m_tiles = m_pad / jq::GD_MT;
    static const char *split_env = getenv("JQ_DECODED_GEMM_SPLITS");
    const size_t splits = m * n / 1024 < 0x7FFFFFFFull ? (size_t)gemm_k_splits(n_tiles * m_tiles, nc, m, n, 5.0, split_env, nullptr, 2 * plane + sbytes) : 1;
    const size_t part_bytes = splits > 1 ? splits * m * n * sizeof(float) : 0;
    CallScratch scratch;
    uint8_t *buf = nullptr;
    if (scratch.get(2 * plane + sbytes + part_bytes, s, &buf)) return 1;
    jq::ActsF16 a{(_Float16 *)buf, (_Float16 *)(buf + plane), (float *)(buf + 2 * plane)};
    float *parts = (float *)(buf + 2 * plane + sbytes);
    note_kernel(splits > 1 ? "gemm_decoded_mfma+splitk" : "gemm_decoded_mfma");
    hipLaunchKernelGGL(jq::acts_f16_prep, dim3((unsigned)((m_pad * nc * 64 + 255) / 256)), dim3(256), 0, s, X, (int)m,
                       (int)m_pad, (int)k, a);
    hipLaunchKernelGGL(jq::gemm_decoded_mfma<Q>, dim3((unsigned)n_tiles, (unsigned)m_tiles, (unsigned)splits), dim3(256), 0, s, W,
                       row_bytes, a, splits > 1 ? parts : Y, (int)m, (int)k, (int)n, splits > 1 ? m * n : (size_t)0);
    if (splits > 1)
        hipLaunchKernelGGL(jq::splitk_sum, dim3((unsigned)((m * n + 1023) / 1024)), dim3(256), 0, s, parts, Y, m * n, (int)splits);
    HIP_TRY(hipGetLastError());
    return 0;
}

int dispatch_gemm_decoded(uint32_t type, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m,
                          size_t k, size_t n, hipStream_t s) {
    switch (type) {
#define JQ_CASE(ID, Q) \
    case ID: return launch_gemm_decoded<jq::Q>(W, row_bytes, X, Y, m, k, n, s);
        JQ_FOR_EACH_FORMAT(JQ_CASE)
#undef JQ_CASE
    default: return -1;
    }
}

// All pointers are device pointers; shapes already validated; m, n > 0.
int dispatch_matmul(uint32_t type, const uint8_t *W, size_t row_bytes, const float *X, float *Y, size_t m,
                    size_t k, size_t n, hipStream_t s) {
    if (m > 0x7FFFFFFF || k > 0x7FFFFFFF || n > 0x7FFFFFFF) return fail("matmul: dimension exceeds 2^31-1");
    if (type == JQ_TYPE_Q4_K && m == 1) {
        const int rc = dispatch_q4k_dot4(W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    if ((type == JQ_TYPE_Q6_K || type == JQ_TYPE_Q8_0) && m == 1) {
        const int rc = dispatch_gemv_tile16(type, W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q6_K && m == 1) {
        const int rc = dispatch_q6k_dot4(W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q2_K && m == 1) {
        const int rc = dispatch_q2k_mfma(W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q8_0 && m == 1) {
        const int rc = dispatch_q8_0_dot4(W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    if (m == 1) {
        int rc = dispatch_gemv_tile8(type, W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
        rc = dispatch_i8_gemv(type, W, row_bytes, X, Y, k, n, s);
        if (rc >= 0) return rc;
    }
    // Q6_K and Q8_0 with two or three activation rows against a matrix of 16M weights or more: the one-row kernel
    // once a row (4096 x 12288 of Q6_K, two rows: 23 us against 28 for the f32 row kernel; the int8 GEMM's 38 us
    // are the same for 2 to 16 rows)
    if ((type == JQ_TYPE_Q6_K || type == JQ_TYPE_Q8_0) && (m == 2 || m == 3) && n * k >= ((size_t)16 << 20)) {
        static const char *no_loop = getenv("JQ_NO_ONE_ROW_LOOP");
        int rc = no_loop ? -1 : 0;
        for (size_t r = 0; r < m && rc == 0; r++)
            rc = type == JQ_TYPE_Q6_K ? dispatch_q6k_dot4(W, row_bytes, X + r * k, Y + r * n, k, n, s)
                                      : dispatch_q8_0_dot4(W, row_bytes, X + r * k, Y + r * n, k, n, s);
        if (rc == 0) return 0;
        if (rc > 0) return rc;  // (a kernel that declines does so at the first row, before anything is launched)
    }
    // Q4_K with a few activation rows.  Rows of 4096, 1024 weight rows or more: the int8 matrix-core kernel
    // on the one-row kernel's weight stream, in passes of 16 activation rows.  Other row lengths: one or two
    // rows on the int8 GEMV further down; from three on the streaming kernel, whose time hardly depends on
    // the row count, or, against a very long matrix (a vocabulary projection), the LDS-ring kernel, whose
    // second launch only pays off from some 100 us of streaming on.
    // (two rows against 2048 to 8192 weight rows of 4096 columns: the one-row kernel twice, 7.6 us at 4096 rows against
    // the 16-row kernel's 9.6 with its preparation launch; from 14336 rows on the two are level and the 16-row kernel
    // reads the matrix once)
    if (type == JQ_TYPE_Q4_K && m == 2 && k == 4096 && n >= 2048 && n <= 8192) {
        static const char *no_loop = getenv("JQ_NO_ONE_ROW_LOOP");
        int rc = no_loop ? -1 : dispatch_q4k_dot4(W, row_bytes, X, Y, k, n, s);
        if (rc == 0) rc = dispatch_q4k_dot4(W, row_bytes, X + k, Y + n, k, n, s);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q4_K && m >= 2) {
        const int rc = dispatch_q4k_rows16(W, row_bytes, X, Y, m, k, n, s);
        if (rc >= 0) return rc;
    }
    static const char *ring_min_env = getenv("JQ_Q4K_RING_MIN_N");
    static const size_t ring_min_n = ring_min_env ? (size_t)atoll(ring_min_env) : 32768;
    if (type == JQ_TYPE_Q4_K && m > 2 && m <= Q4K_MFMA_MAX_M && n >= ring_min_n) {
        const int rc = dispatch_q4k_ring(W, row_bytes, X, Y, m, k, n, s);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q4_K && m > 2 && m <= Q4K_MFMA_MAX_M) {
        const int rc = dispatch_q4k_stream(W, row_bytes, X, Y, m, k, n, s);
        if (rc >= 0) return rc;
    }
    // rows longer than 4096 with 3..16 activation rows: the int8 GEMV below walks the matrix once per two
    // rows (6.5 us a row at 4096 x 12288); from where that exceeds the estimate of the GEMM split over k
    // (48 us there at any of these row counts), the GEMM
    const bool gemm_ok = type == JQ_TYPE_Q4_K && row_bytes % 16 == 0 && ((uintptr_t)W & 15) == 0 && !getenv("JQ_Q4K_NO_GEMM");
    if (gemm_ok && m > 2 && m <= Q4K_MFMA_MAX_M && k > 4096 &&
        q4k_gemm_estimate_us(m, k, n) < (double)m * (2.0 + (double)n * (double)row_bytes / 4.0e6))
        return dispatch_q4k_gemm(W, row_bytes, X, Y, m, k, n, s);
    if (type == JQ_TYPE_Q4_K && q4k_mfma_applies(m, k, n)) return dispatch_q4k_mfma(W, row_bytes, X, Y, m, k, n, s);
    if (type == JQ_TYPE_Q4_K && m > Q4K_MFMA_MAX_M) {
        const int rc = dispatch_gemm_i8<jq::QiQ4K>(W, row_bytes, X, Y, m, k, n, s, "q4k_gemm_i8", "q4k_gemm_i8+splitk");
        if (rc >= 0) return rc;
    }
    // every other format (Q6_K, Q2_K, Q8_0, IQ2_XXS, MXFP4, Q5_K, Q4_0, Q3_K, Q5_0, Q4_1, Q5_1): the same GEMM wherever the MFMA GEMM over decoded weights would run otherwise (from 17
    // rows on, and from JQ_DECODED_GEMM_MIN_M rows on against matrices of 8M elements or more)
    static const char *dec_min_m_env = getenv("JQ_DECODED_GEMM_MIN_M");
    static const size_t gemm_min_m = dec_min_m_env ? (size_t)std::max(atoi(dec_min_m_env), 2) : 8;
    // (the f32 row kernel's time grows with the row count, 12 us a row against 50M weights of Q6_K, the GEMM's does
    // not: 38 us there, 22 us against 16M; it takes over from 4 rows against 32M weights or more, from 6 against 8M)
    const size_t min_m = dec_min_m_env ? gemm_min_m : n * k >= ((size_t)32 << 20) ? 4 : 6;
    const bool many_rows = m > Q4K_MFMA_MAX_M || (m >= min_m && n * k >= ((size_t)8 << 20));
    if (type == JQ_TYPE_Q6_K && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ6K>(W, row_bytes, X, Y, m, k, n, s, "q6k_gemm_i8", "q6k_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q2_K && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ2K>(W, row_bytes, X, Y, m, k, n, s, "q2k_gemm_i8", "q2k_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q8_0 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ8_0>(W, row_bytes, X, Y, m, k, n, s, "q8_0_gemm_i8", "q8_0_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_IQ2_XXS && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiIQ2XXS>(W, row_bytes, X, Y, m, k, n, s, "iq2xxs_gemm_i8", "iq2xxs_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q5_K && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ5K>(W, row_bytes, X, Y, m, k, n, s, "q5k_gemm_i8", "q5k_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q3_K && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ3K>(W, row_bytes, X, Y, m, k, n, s, "q3k_gemm_i8", "q3k_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q5_0 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ5_0>(W, row_bytes, X, Y, m, k, n, s, "q5_0_gemm_i8", "q5_0_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q4_1 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ4_1>(W, row_bytes, X, Y, m, k, n, s, "q4_1_gemm_i8", "q4_1_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q5_1 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ5_1>(W, row_bytes, X, Y, m, k, n, s, "q5_1_gemm_i8", "q5_1_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q4_0 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiQ4_0>(W, row_bytes, X, Y, m, k, n, s, "q4_0_gemm_i8", "q4_0_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_MXFP4 && many_rows) {
        const int rc = dispatch_gemm_i8<jq::QiMXFP4>(W, row_bytes, X, Y, m, k, n, s, "mxfp4_gemm_i8", "mxfp4_gemm_i8+splitk", false, 2);
        if (rc >= 0) return rc;
    }
    if (type == JQ_TYPE_Q4_K && m > Q4K_MFMA_MAX_M && row_bytes % 16 == 0 && ((uintptr_t)W & 15) == 0 &&
        !getenv("JQ_Q4K_NO_GEMM"))
        return dispatch_q4k_gemm(W, row_bytes, X, Y, m, k, n, s);
    // the other formats: the MFMA GEMM over decoded weights from 17 rows on, and (split over k, its 64-row
    // activation tile part empty) from JQ_DECODED_GEMM_MIN_M rows (default 8) on against matrices of 8M
    // elements or more, where the f32 staged kernel takes a pass over the matrix per four rows (Q6_K
    // 4096 x 12288: 77 us at any row count against 92 us at 8 rows and 178 us at 16)
    if (many_rows && type != JQ_TYPE_Q4_K) {
        const int rc = dispatch_gemm_decoded(type, W, row_bytes, X, Y, m, k, n, s);
        if (rc >= 0) return rc;
    }
    switch (type) {
#define JQ_CASE(ID, Q) \
    case ID: launch_rows<jq::Q>(W, row_bytes, X, Y, m, k, n, s); break;
        JQ_FOR_EACH_FORMAT(JQ_CASE)
#undef JQ_CASE
    default: return fail("unsupported tensor type id %u", type);
    }
    HIP_TRY(hipGetLastError());
    return 0;
}

template <class Q>
void launch_decode(const jq_weight *w, const uint32_t *ids, float *out, size_t rows, hipStream_t s) {
    size_t units = rows * (w->k / Q::BLOCK_ELEMS) * Q::UNITS;
    unsigned blocks = (unsigned)std::min<size_t>((units + 255) / 256, 65535u * 16u);
    if (blocks == 0) return;
    hipLaunchKernelGGL((jq::decode_rows<Q>), dim3(blocks), dim3(256), 0, s, w->dev, w->row_bytes, ids, out, rows,
                       (int)w->k);
}

int dispatch_decode(const jq_weight *w, const uint32_t *ids, float *out, size_t rows, hipStream_t s) {
    switch (w->type) {
#define JQ_CASE(ID, Q) \
    case ID: launch_decode<jq::Q>(w, ids, out, rows, s); break;
        JQ_FOR_EACH_FORMAT(JQ_CASE)
#undef JQ_CASE
    default: return fail("unsupported tensor type id %u", w->type);
    }
    HIP_TRY(hipGetLastError());
    return 0;
}

// Frees a device allocation when it goes out of scope.
struct DevBuf {
    void *p = nullptr;
    ~DevBuf() {
        if (p) (void)hipFree(p);
    }
    hipError_t alloc(size_t bytes) { return hipMalloc(&p, bytes ? bytes : 1); }
};

}  // namespace

extern "C" {

const char *jq_last_error(void) { return g_err; }
const char *jq_last_kernel(void) { return g_last_kernel; }

int jq_block_geometry(uint32_t ggml_type, size_t *elems, size_t *bytes) {
    Geometry g;
    if (!geometry(ggml_type, &g)) return fail("unsupported tensor type id %u", ggml_type);
    if (elems) *elems = g.elems;
    if (bytes) *bytes = g.bytes;
    return 0;
}

int jq_init(int device) {
    bool first = false;
    std::call_once(g_init_once, [&] {
        first = true;
        g_init_rc = do_init(device);
    });
    if (!first && g_init_rc == 0 && device != g_device)
        return fail("jq_init: already initialised on device %d", g_device);
    return g_init_rc;
}

int jq_upload(uint32_t ggml_type, const void *blocks, size_t nbytes, size_t n, size_t k, int src_is_device,
              jq_weight **out) {
    if (!out) return fail("jq_upload: out is null");
    *out = nullptr;
    Geometry g;
    if (!geometry(ggml_type, &g)) return fail("unsupported tensor type id %u", ggml_type);
    if (k % g.elems != 0)
        return fail("%s tensor: k=%zu is not a multiple of the block size %zu", type_name(ggml_type), k, g.elems);
    size_t want = n * (k / g.elems) * g.bytes;
    if (nbytes != want)
        return fail("%s tensor: %zu bytes for %zu x %zu elements (expected %zu)", type_name(ggml_type), nbytes, n, k,
                    want);
    if (nbytes && !blocks) return fail("jq_upload: blocks is null");
    if (ensure_init()) return 1;
    uint8_t *dev = nullptr;
    // Kernels read a row in 16-byte pieces that may start before the unit they
    // need; 64 spare bytes keep every such read inside the allocation.
    HIP_TRY(hipMalloc((void **)&dev, nbytes + 64));
    hipError_t e = hipMemcpy(dev, blocks, nbytes, src_is_device ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice);
    if (e == hipSuccess) e = hipMemset(dev + nbytes, 0, 64);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return fail("jq_upload: copy to device failed: %s", hipGetErrorString(e));
    }
    *out = new jq_weight{ggml_type, n, k, nbytes, (k / g.elems) * g.bytes, dev, true};
    return 0;
}

int jq_view(const jq_weight *parent, size_t byte_offset, size_t n, size_t k, jq_weight **out) {
    if (!out) return fail("jq_view: out is null");
    *out = nullptr;
    if (!parent) return fail("jq_view: parent is null");
    Geometry g;
    geometry(parent->type, &g);
    if (k % g.elems != 0)
        return fail("%s tensor: k=%zu is not a multiple of the block size %zu", type_name(parent->type), k, g.elems);
    size_t need = n * (k / g.elems) * g.bytes;
    // reference: src/mmap_tensor.rs:105-110 (range must lie inside the mapping)
    if (byte_offset > parent->nbytes || need > parent->nbytes - byte_offset)
        return fail("jq_view: range %zu+%zu exceeds the parent's %zu bytes", byte_offset, need, parent->nbytes);
    if (byte_offset % g.bytes != 0) return fail("jq_view: offset %zu is not a whole number of blocks", byte_offset);
    *out = new jq_weight{parent->type, n, k, need, (k / g.elems) * g.bytes, parent->dev + byte_offset, false};
    return 0;
}

void jq_free(jq_weight *w) {
    if (!w) return;
    if (w->owns && w->dev) (void)hipFree(w->dev);
    delete w;
}

uint32_t jq_dtype(const jq_weight *w) { return w ? w->type : 0; }
size_t jq_rows(const jq_weight *w) { return w ? w->n : 0; }
size_t jq_cols(const jq_weight *w) { return w ? w->k : 0; }
size_t jq_storage_size_in_bytes(const jq_weight *w) { return w ? w->nbytes : 0; }
const void *jq_device_ptr(const jq_weight *w) { return w ? w->dev : nullptr; }

int jq_matmul_t(const jq_weight *w, size_t m, const float *lhs, size_t lhs_len, float *dst, size_t dst_len,
                int ptrs_are_device, void *stream) {
    if (!w) return fail("jq_matmul_t: weight is null");
    if (validate(w->type, m, w->k, w->n, lhs_len, w->nbytes, dst_len)) return 1;
    if (m == 0 || w->n == 0) return 0;  // reference: src/quant_matmul.rs:176-178
    if (!lhs || !dst) return fail("jq_matmul_t: lhs/dst is null");
    hipStream_t s = (hipStream_t)stream;
    if (ptrs_are_device) return dispatch_matmul(w->type, w->dev, w->row_bytes, lhs, dst, m, w->k, w->n, s);
    DevBuf x, y;
    HIP_TRY(x.alloc(lhs_len * sizeof(float)));
    HIP_TRY(y.alloc(dst_len * sizeof(float)));
    HIP_TRY(hipMemcpyAsync(x.p, lhs, lhs_len * sizeof(float), hipMemcpyHostToDevice, s));
    if (dispatch_matmul(w->type, w->dev, w->row_bytes, (const float *)x.p, (float *)y.p, m, w->k, w->n, s)) return 1;
    HIP_TRY(hipMemcpyAsync(dst, y.p, dst_len * sizeof(float), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int jq_matmul_t_f16(const jq_weight *w, size_t m, const uint16_t *lhs, size_t lhs_len, uint16_t *dst, size_t dst_len,
                    int ptrs_are_device, void *stream) {
    if (!w) return fail("jq_matmul_t_f16: weight is null");
    if (validate(w->type, m, w->k, w->n, lhs_len, w->nbytes, dst_len)) return 1;
    if (m == 0 || w->n == 0) return 0;
    if (!lhs || !dst) return fail("jq_matmul_t_f16: lhs/dst is null");
    hipStream_t s = (hipStream_t)stream;
    // f16 -> f32, the f32 product, f32 -> f16 (reference: src/mxfp4.rs:242-258, src/iq2xxs.rs:396-412): the f32
    // operands live in the stream's second kept buffer (up to 64 MB; a stream-ordered allocation beyond), so
    // device callers are not synchronised and a call on a warmed-up stream allocates nothing
    const size_t h16_bytes = ptrs_are_device ? 0 : std::max(lhs_len, dst_len) * sizeof(uint16_t);
    const size_t x_bytes = (lhs_len * sizeof(float) + 255) & ~(size_t)255, y_bytes = (dst_len * sizeof(float) + 255) & ~(size_t)255;
    CallScratch stage(1);
    uint8_t *base = nullptr;
    if (stage.get(x_bytes + y_bytes + h16_bytes, s, &base)) return 1;
    float *x32 = (float *)base, *y32 = (float *)(base + x_bytes);
    uint16_t *h16 = (uint16_t *)(base + x_bytes + y_bytes);
    if (!ptrs_are_device) HIP_TRY(hipMemcpyAsync(h16, lhs, lhs_len * sizeof(uint16_t), hipMemcpyHostToDevice, s));
    const uint16_t *x16 = ptrs_are_device ? lhs : (const uint16_t *)h16;
    uint16_t *y16 = ptrs_are_device ? dst : h16;
    auto grid_of = [](size_t elems) { return (unsigned)std::min<size_t>((elems + 255) / 256, 65536); };
    hipLaunchKernelGGL((jq::decode_plain<1>), dim3(grid_of(lhs_len)), dim3(256), 0, s, (const uint8_t *)x16, x32, lhs_len);
    if (dispatch_matmul(w->type, w->dev, w->row_bytes, x32, y32, m, w->k, w->n, s)) return 1;
    hipLaunchKernelGGL(jq::f32_to_f16, dim3(grid_of(dst_len)), dim3(256), 0, s, (const float *)y32, y16, dst_len);
    HIP_TRY(hipGetLastError());
    if (!ptrs_are_device) {
        HIP_TRY(hipMemcpyAsync(dst, h16, dst_len * sizeof(uint16_t), hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    return 0;
}

int jq_matmul_t_noalloc(const jq_weight *w, size_t m, const float *lhs_dev, size_t lhs_len, float *dst_dev,
                        size_t dst_len, void *stream) {
    if (!w) return fail("jq_matmul_t_noalloc: weight is null");
    if (validate(w->type, m, w->k, w->n, lhs_len, w->nbytes, dst_len)) return 1;
    if (m == 0 || w->n == 0) return 0;
    if (!lhs_dev || !dst_dev) return fail("jq_matmul_t_noalloc: lhs/dst is null");
    int dev = 0;
    HIP_TRY(hipGetDevice(&dev));
    FixedScratch f;
    if (noalloc_scratch_on(dev, &f.ptr)) return 1;  // resolved by jq_init; the first call on another device resolves it there
    f.bytes = JQ_NOALLOC_SCRATCH_BYTES;
    f.mu = &g_scratch_mu[dev];
    FixedScratchScope scope(&f);
    return dispatch_matmul(w->type, w->dev, w->row_bytes, lhs_dev, dst_dev, m, w->k, w->n, (hipStream_t)stream);
}

int jq_try_matmul_fused(uint32_t ggml_type, size_t m, size_t k, size_t n, const float *lhs_dev,
                        const void *blocks_dev, size_t nbytes, float *dst_dev, void *stream) {
    Geometry g;
    // reference: src/kquant_dot.rs:158-163 (unknown dtype declines),
    // :217-224 (ragged byte length or k shorter than a block declines)
    if (!geometry(ggml_type, &g)) return fail("declined: no fused kernel for tensor type id %u", ggml_type);
    if (nbytes % g.bytes != 0) return fail("declined: %zu bytes is not a whole number of %zu byte blocks", nbytes, g.bytes);
    if (k / g.elems == 0 || k % g.elems != 0) return fail("declined: k=%zu is not a positive multiple of %zu", k, g.elems);
    if (nbytes / g.bytes != n * (k / g.elems))
        return fail("declined: rhs holds %zu blocks, expected %zu", nbytes / g.bytes, n * (k / g.elems));
    if (m == 0 || n == 0) return 0;
    if (!lhs_dev || !blocks_dev || !dst_dev) return fail("declined: null pointer");
    if (ensure_init()) return 1;
    return dispatch_matmul(ggml_type, (const uint8_t *)blocks_dev, (k / g.elems) * g.bytes, lhs_dev, dst_dev, m, k, n,
                           (hipStream_t)stream);
}

int jq_stream_release(void *stream) {
    if (ensure_init()) return 1;
    return release_stream_scratch((hipStream_t)stream);
}

int jq_dequantize(const jq_weight *w, float *out, size_t out_len, int out_is_device, void *stream) {
    if (!w) return fail("jq_dequantize: weight is null");
    if (out_len != w->n * w->k)
        return fail("%s: output holds %zu values, expected %zu", type_name(w->type), out_len, w->n * w->k);
    if (out_len == 0) return 0;
    if (!out) return fail("jq_dequantize: out is null");
    hipStream_t s = (hipStream_t)stream;
    if (out_is_device) return dispatch_decode(w, nullptr, out, w->n, s);
    DevBuf y;
    HIP_TRY(y.alloc(out_len * sizeof(float)));
    if (dispatch_decode(w, nullptr, (float *)y.p, w->n, s)) return 1;
    HIP_TRY(hipMemcpyAsync(out, y.p, out_len * sizeof(float), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int jq_decode_raw_to_f32(uint32_t ggml_type, const void *bytes, size_t nbytes, size_t elems, float *out,
                         int ptrs_are_device, void *stream) {
    if (ggml_type == 0) return 2;  // F32: the caller's own reader keeps it exact
    const bool plain = ggml_type == 1 || ggml_type == 9 || ggml_type == 15;
    size_t blck = 1, bb = 2;
    if (ggml_type == 9) blck = 32, bb = 36;
    else if (ggml_type == 15) blck = 256, bb = 292;
    else if (!plain) {
        Geometry g;
        if (!geometry(ggml_type, &g)) return 2;  // no decoder in the reference either: Ok(None)
        blck = g.elems, bb = g.bytes;
    }
    if (ggml_type == 16 || ggml_type == 39) {
        // the in-mapping formats fail in their own block readers, with their own words
        // (src/iq2xxs.rs:75-82,422-429, src/mxfp4.rs:99-106,265-272; the output there is sized by `elems`)
        const char *nm = ggml_type == 16 ? "iq2_xxs" : "mxfp4";
        if (nbytes % bb != 0)
            return fail(ggml_type == 16 ? "%s: %zu bytes is not a whole number of %zu byte blocks" : "%s: %zu bytes is not a whole number of %zu-byte blocks", nm, nbytes, bb);
        if (elems != nbytes / bb * blck) return fail("%s: output holds %zu values, expected %zu", nm, elems, nbytes / bb * blck);
    }
    if (elems % blck != 0 || nbytes != elems / blck * bb) {
        if (ggml_type == 1) return fail("dtype F16: %zu bytes for %zu elements", nbytes, elems);
        return fail("dtype %u: %zu bytes for %zu elements (%zu per %zu-block)", ggml_type, nbytes, elems, bb, blck);
    }
    if (elems == 0) return 0;
    if (!bytes || !out) return fail("jq_decode_raw_to_f32: null pointer");
    if (ensure_init()) return 1;
    hipStream_t s = (hipStream_t)stream;
    DevBuf in, y;
    const uint8_t *src = (const uint8_t *)bytes;
    float *dst = out;
    if (!ptrs_are_device) {
        HIP_TRY(in.alloc(nbytes));
        HIP_TRY(y.alloc(elems * sizeof(float)));
        HIP_TRY(hipMemcpyAsync(in.p, bytes, nbytes, hipMemcpyHostToDevice, s));
        src = (const uint8_t *)in.p, dst = (float *)y.p;
    }
    if (plain) {
        const unsigned blocks = (unsigned)std::min<size_t>((elems + 255) / 256, 65535u * 16u);
        if (ggml_type == 1) hipLaunchKernelGGL((jq::decode_plain<1>), dim3(blocks), dim3(256), 0, s, src, dst, elems);
        else if (ggml_type == 9) hipLaunchKernelGGL((jq::decode_plain<9>), dim3(blocks), dim3(256), 0, s, src, dst, elems);
        else hipLaunchKernelGGL((jq::decode_plain<15>), dim3(blocks), dim3(256), 0, s, src, dst, elems);
        HIP_TRY(hipGetLastError());
    } else {
        // The block decoders index a row's columns with an int, so the caller's bytes are decoded as rows of at
        // most 2^20 blocks (a tensor of 2^31 elements or more, a stacked expert tensor, is many such rows and a
        // shorter last one).  JQ_DECODE_CHUNK_BLOCKS, read at every call, sets another row length (for tests).
        size_t chunk_max = (size_t)1 << 20;
        if (const char *env = getenv("JQ_DECODE_CHUNK_BLOCKS")) chunk_max = std::max<size_t>(1, (size_t)atoll(env));
        const size_t blocks_total = elems / blck;
        for (size_t b0 = 0; b0 < blocks_total;) {
            const size_t left = blocks_total - b0;
            const size_t rows = left >= chunk_max ? left / chunk_max : 1, per = left >= chunk_max ? chunk_max : left;
            jq_weight view{};
            view.type = ggml_type, view.dev = const_cast<uint8_t *>(src) + b0 * bb, view.n = rows, view.k = per * blck, view.row_bytes = per * bb;
            if (dispatch_decode(&view, nullptr, dst + b0 * blck, rows, s)) return 1;
            b0 += rows * per;
        }
    }
    if (!ptrs_are_device) {
        HIP_TRY(hipMemcpyAsync(out, y.p, elems * sizeof(float), hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    return 0;
}

int jq_embedding(const jq_weight *w, const uint32_t *ids, size_t n_ids, float *out, size_t out_len,
                 int ptrs_are_device, void *stream) {
    if (!w) return fail("jq_embedding: weight is null");
    if (out_len != n_ids * w->k)
        return fail("quantized embedding: output holds %zu values, expected %zu", out_len, n_ids * w->k);
    if (n_ids == 0) return 0;
    if (!ids || !out) return fail("jq_embedding: ids/out is null");
    hipStream_t s = (hipStream_t)stream;
    // The id check happens on the host, as in the reference
    // (src/mmap_tensor.rs:157-161); device-resident ids are read back for it.
    std::vector<uint32_t> host_ids;
    const uint32_t *check = ids;
    if (ptrs_are_device) {
        host_ids.resize(n_ids);
        HIP_TRY(hipMemcpyAsync(host_ids.data(), ids, n_ids * sizeof(uint32_t), hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
        check = host_ids.data();
    }
    for (size_t i = 0; i < n_ids; i++)
        if (check[i] >= w->n) return fail("embedding id %u is out of range for %zu rows", check[i], w->n);
    if (ptrs_are_device) return dispatch_decode(w, ids, out, n_ids, s);
    DevBuf di, y;
    HIP_TRY(di.alloc(n_ids * sizeof(uint32_t)));
    HIP_TRY(y.alloc(out_len * sizeof(float)));
    HIP_TRY(hipMemcpyAsync(di.p, ids, n_ids * sizeof(uint32_t), hipMemcpyHostToDevice, s));
    if (dispatch_decode(w, (const uint32_t *)di.p, (float *)y.p, n_ids, s)) return 1;
    HIP_TRY(hipMemcpyAsync(out, y.p, out_len * sizeof(float), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int jq_stream_synchronize(void *stream) {
    HIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}


// ---- mixture of experts -----------------------------------------------------------

}  // extern "C"

struct jq_moe {
    jq_moe_config cfg;
    const jq_weight *gate, *up, *down, *sgate, *sup, *sdown;
    float *router_w = nullptr, *router_bias = nullptr;
    const uint8_t **pgate = nullptr, **pup = nullptr, **pdown = nullptr;  // device tables of expert bases
    bool fold_shared = false;  // the shared expert rides along as table entry n_expert of the grouped kernels
    // scratch, grown to the largest token count seen
    size_t cap_tokens = 0;
    float *logits = nullptr, *wts = nullptr, *G = nullptr, *U = nullptr, *out = nullptr;
    float *sG = nullptr, *sU = nullptr, *sH = nullptr, *sOut = nullptr;
    uint32_t *ids = nullptr;
    int *gexp = nullptr, *offsets = nullptr, *xrow = nullptr, *yrow = nullptr;
    uint8_t *qacts = nullptr;  // activations as MFMA operand records (Q4_K experts, grouped path)
    uint8_t *gacts = nullptr;  // activations of the grouped int8 GEMM, and its tables
    int *gtab = nullptr;
    size_t gtab_rows = 0;      // row groups (and tiles) the tables hold
    int gtile_rgs = 8;         // row groups a tile of the current plan: 8 (waves share the rows), 2 (the weight rows), 0 (both: two launches)
    jq::ActsI8 qi8{nullptr, nullptr, nullptr, nullptr};  // activations as int8 planes (decode path, long rows)
    std::mutex mu;
};

namespace {

void moe_free_scratch(jq_moe *m) {
    for (void *p : {(void *)m->logits, (void *)m->wts, (void *)m->G, (void *)m->U, (void *)m->out, (void *)m->sG,
                    (void *)m->sU, (void *)m->sH, (void *)m->sOut, (void *)m->ids, (void *)m->gexp,
                    (void *)m->offsets, (void *)m->xrow, (void *)m->yrow, (void *)m->qacts, (void *)m->qi8.xl,
                    (void *)m->qi8.xh, (void *)m->qi8.sx, (void *)m->qi8.sxs, (void *)m->gacts, (void *)m->gtab})
        if (p) (void)hipFree(p);
    m->qacts = nullptr;
    m->gacts = nullptr, m->gtab = nullptr, m->gtab_rows = 0;
    m->qi8 = jq::ActsI8{nullptr, nullptr, nullptr, nullptr};
    m->logits = m->wts = m->G = m->U = m->out = m->sG = m->sU = m->sH = m->sOut = nullptr;
    m->ids = nullptr;
    m->gexp = m->offsets = m->xrow = m->yrow = nullptr;
    m->cap_tokens = 0;
}

// Formats whose decode-shaped expert matmuls run on integer dot products (Q::dot8).
bool moe_has_dot8(uint32_t type) {
    static const char *env = getenv("JQ_MOE_DOT8");  // "0": none; a list of type ids ("39,16"): those only
    if (type != JQ_TYPE_MXFP4 && type != JQ_TYPE_IQ2_XXS && type != JQ_TYPE_Q4_K) return false;
    if (!env) return true;
    const std::string list = std::string(",") + env + ",";
    return list.find("," + std::to_string(type) + ",") != std::string::npos;
}

// Formats whose units decode to signed int8 words (Q::decode_i8): bucketed calls of few pairs an expert can
// run on moe_expert_dot8.
bool moe_has_decode_i8(uint32_t type) {
    return (type == JQ_TYPE_MXFP4 || type == JQ_TYPE_IQ2_XXS || type == JQ_TYPE_Q4_K) && moe_has_dot8(type);
}

// Formats with a side of the int8 GEMM (kq_gemm_i8): their grouped expert matmuls run on it.
bool moe_has_gemm_i8(uint32_t type) {
    static const char *off = getenv("JQ_MOE_NO_GEMM_I8");
    if (off) return false;
    return type == JQ_TYPE_Q4_K || type == JQ_TYPE_Q6_K || type == JQ_TYPE_Q2_K || type == JQ_TYPE_Q8_0 ||
           type == JQ_TYPE_IQ2_XXS || type == JQ_TYPE_MXFP4 || type == JQ_TYPE_Q5_K || type == JQ_TYPE_Q4_0 || type == JQ_TYPE_Q3_K || type == JQ_TYPE_Q5_0 || type == JQ_TYPE_Q4_1 ||
           type == JQ_TYPE_Q5_1;
}

int moe_reserve(jq_moe *m, size_t T) {
    if (T <= m->cap_tokens) return 0;
    moe_free_scratch(m);
    const jq_moe_config &c = m->cfg;
    // rows of the pair buffers: the routed pairs, then one per token for a folded shared expert
    size_t P = T * c.n_expert_used, PR = P + T, groups = std::max<size_t>(PR, c.n_expert + 1) + 1;
    HIP_TRY(hipMalloc((void **)&m->logits, T * c.n_expert * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->wts, P * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->ids, P * sizeof(uint32_t)));
    HIP_TRY(hipMalloc((void **)&m->G, PR * c.inter * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->U, PR * c.inter * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->out, PR * c.hidden * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->gexp, groups * sizeof(int)));
    HIP_TRY(hipMalloc((void **)&m->offsets, (groups + 1) * sizeof(int)));
    HIP_TRY(hipMalloc((void **)&m->xrow, PR * sizeof(int)));
    HIP_TRY(hipMalloc((void **)&m->yrow, PR * sizeof(int)));
    if (moe_has_dot8(m->gate->type) || moe_has_dot8(m->down->type)) {
        const size_t words = PR * (std::max<size_t>(c.hidden, c.inter) / 4);
        HIP_TRY(hipMalloc((void **)&m->qi8.xl, words * sizeof(uint32_t) + 16));
        HIP_TRY(hipMalloc((void **)&m->qi8.xh, words * sizeof(uint32_t) + 16));
        HIP_TRY(hipMalloc((void **)&m->qi8.sx, (words / 8 + 1) * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&m->qi8.sxs, (words / 8 + 1) * sizeof(float)));
    }
    if (m->gate->type == JQ_TYPE_Q4_K || m->down->type == JQ_TYPE_Q4_K)
        HIP_TRY(hipMalloc((void **)&m->qacts, std::max(T * (c.hidden / 256), PR * (c.inter / 256)) * jq::QS_REC + 16));
    if (P > c.n_expert && (moe_has_gemm_i8(m->gate->type) || moe_has_gemm_i8(m->down->type))) {
        // row groups of 16 pairs that never mix two experts: at most PR / 16 + one part-filled group an expert
        m->gtab_rows = PR / 16 + c.n_expert + 2;
        HIP_TRY(hipMalloc((void **)&m->gacts, m->gtab_rows * (std::max<size_t>(c.hidden, c.inter) / 256 + 1) * jq::QI_REC));
        HIP_TRY(hipMalloc((void **)&m->gtab, (8 * m->gtab_rows + 4) * sizeof(int)));
    }
    if (m->sgate) {
        size_t si = m->sgate->n;
        HIP_TRY(hipMalloc((void **)&m->sG, T * si * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&m->sU, T * si * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&m->sH, T * si * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&m->sOut, T * c.hidden * sizeof(float)));
    }
    m->cap_tokens = T;
    return 0;
}

template <class Q, bool SWIGLU>
void launch_moe_rows(const uint8_t *const *Wptr, size_t row_bytes, const float *X, const float *X2, const int *gexp,
                     const int *offsets, const int *xsel, const int *yrow, float *Y, int k, int n, int groups,
                     int max_group, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    dim3 grid((unsigned)((n + jq::ROWS_PER_WG - 1) / jq::ROWS_PER_WG), (unsigned)groups), block(64 * jq::ROWS_PER_WG);
    if (max_group <= 1)
        hipLaunchKernelGGL((jq::moe_rows_valu<Q, 1, SWIGLU>), grid, block, 0, s, Wptr, row_bytes, X, X2, gexp, offsets,
                           xsel, yrow, Y, k, n, cl);
    else
        hipLaunchKernelGGL((jq::moe_rows_valu<Q, 4, SWIGLU>), grid, block, 0, s, Wptr, row_bytes, X, X2, gexp, offsets,
                           xsel, yrow, Y, k, n, cl);
}

// The LDS-staged grouped kernel when the rows allow it (aligned row starts, four waves' rows within
// 64 KB); returns -1 when they do not and the caller takes the plain kernels.
template <class Q, bool DUAL>
int launch_moe_staged(const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align,
                      const float *X, const int *gexp, const int *offsets, const int *xsel, const int *yrow, float *Y,
                      int k, int n, int groups, int max_group, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    const int L = units >= 48 ? 64 : units >= 24 ? 32 : 16, R = 64 / L;
    const int G = (row_bytes % 16 == 0 && base_align >= 16) ? 16 : (row_bytes % 4 == 0 && base_align >= 4) ? 4 : 0;
    const size_t one = ((size_t)R * row_bytes + 15) / 16 * 16, wave_lds = one * (DUAL ? 2 : 1);
    if (G == 0 || wave_lds * jq::ROWS_PER_WG + jq::table_bytes<Q>() > 64 * 1024 || getenv("JQ_NO_STAGED_ROWS")) return -1;
    dim3 grid((unsigned)((n + jq::ROWS_PER_WG * R - 1) / (jq::ROWS_PER_WG * R)), (unsigned)groups), block(64 * jq::ROWS_PER_WG);
    const size_t lds = wave_lds * jq::ROWS_PER_WG + jq::table_bytes<Q>();
#define JQ_MOE_STAGED(MT, GG)                                                                                      \
    hipLaunchKernelGGL((jq::moe_rows_staged<Q, MT, DUAL, GG>), grid, block, lds, s, Wa, Wb, row_bytes, X, gexp,     \
                       offsets, xsel, yrow, Y, k, n, L, (int)wave_lds, cl)
    if (max_group <= 1) {
        if (G == 16) JQ_MOE_STAGED(1, 16);
        else JQ_MOE_STAGED(1, 4);
    } else {
        if (G == 16) JQ_MOE_STAGED(4, 16);
        else JQ_MOE_STAGED(4, 4);
    }
#undef JQ_MOE_STAGED
    return 0;
}

template <bool DUAL>
int dispatch_moe_staged(uint32_t type, const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes,
                        int base_align, const float *X, const int *gexp, const int *offsets, const int *xsel,
                        const int *yrow, float *Y, int k, int n, int groups, int max_group, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    int rc;
    switch (type) {
#define JQ_MOE_CASE(ID, Q)                                                                                          \
    case ID:                                                                                                        \
        rc = launch_moe_staged<jq::Q, DUAL>(Wa, Wb, row_bytes, base_align, X, gexp, offsets, xsel, yrow, Y, k, n,     \
                                            groups, max_group, s, cl);                                              \
        break;
        JQ_FOR_EACH_FORMAT(JQ_MOE_CASE)
#undef JQ_MOE_CASE
    default: return fail("unsupported tensor type id %u", type);
    }
    if (rc == 0) HIP_TRY(hipGetLastError());
    return rc;
}

// Q4_K experts with several tokens per group: the LDS-ring MFMA kernel per group.
// Returns -1 when the shape is outside its reach.
template <bool DUAL>
int dispatch_moe_q4k_ring(const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align,
                          const float *X, size_t x_rows, uint8_t *acts, const int *gexp, const int *offsets,
                          const int *xsel, const int *yrow, float *Y, int k, int n, int groups, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    const int nb = k / 256;
    static const char *off = getenv("JQ_MOE_NO_RING");
    if (off || !acts || k % 256 != 0 || nb == 0 || nb > 16 || row_bytes != (size_t)nb * 144 || base_align < 16 ||
        ((uintptr_t)X & 15) != 0)
        return -1;
    launch_q4k_acts_prep(X, x_rows, (size_t)k, acts, s);
    const int maxnb = nb > 8 ? 16 : nb > 4 ? 8 : 4, n_tiles = (n + 15) / 16;
    static const char *genv = getenv("JQ_MOE_RING_GRID");
    const int per_group = genv ? atoi(genv) : 1024 / std::max(groups, 1);
    dim3 grid((unsigned)std::min(n_tiles, std::max(per_group, 1)), (unsigned)groups), block(64 * nb);
#define JQ_RING(MAXNB)                                                                                             \
    hipLaunchKernelGGL((jq::q4k_ring_mfma<MAXNB, true, DUAL>), grid, block, 0, s, nullptr, Wa, Wb, acts, gexp,     \
                       offsets, xsel, yrow, Y, 0, n, cl)
    if (maxnb == 16) JQ_RING(16);
    else if (maxnb == 8) JQ_RING(8);
    else JQ_RING(4);
#undef JQ_RING
    HIP_TRY(hipGetLastError());
    return 0;
}

// Q4_K experts with a few tokens per group (four on average at batch 64 over 128 experts): the int8 kernel
// that multiplies four activation rows an MFMA.  Returns -1 when the shape is outside its reach.
bool moe_q4k_quads_takes(const jq::ActsI8 &xq, size_t row_bytes, int base_align, const float *X, int k) {
    const int nb = k / 256;
    static const char *off = getenv("JQ_MOE_NO_QUADS");
    return !(off || !xq.xl || k % 256 != 0 || nb < 2 || nb > 16 || row_bytes != (size_t)nb * 144 || base_align < 16 ||
             ((uintptr_t)X & 15) != 0);
}

template <bool DUAL>
int dispatch_moe_q4k_quads(const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align,
                           const float *X, size_t x_rows, jq::ActsI8 xq, const int *gexp, const int *offsets,
                           const int *xsel, const int *yrow, float *Y, int k, int n, int groups, hipStream_t s,
                           const jq::MoeClamp &cl = jq::MoeClamp{}, bool planes_ready = false) {
    const int nb = k / 256;
    if (!moe_q4k_quads_takes(xq, row_bytes, base_align, X, k)) return -1;
    const size_t words = x_rows * (size_t)(k / 4);
    if (!planes_ready)  // (else the router launch left X as planes in xq)
        hipLaunchKernelGGL(jq::acts_i8_prep, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, X, x_rows, k, xq);
    const int maxnb = nb > 8 ? 16 : nb > 4 ? 8 : 4, n_tiles = (n + 15) / 16;
    // 2048 workgroups a launch (measured at 128 groups of 768 x 2048: 8 a group 184 us a layer call, 16: 173,
    // 24: 177, 48: 202; the f16 ring kernel: 204 at 8 and more above)
    static const char *genv = getenv("JQ_MOE_QUADS_GRID");
    const int per_group = genv ? atoi(genv) : 2048 / std::max(groups, 1);
    dim3 grid((unsigned)std::min(n_tiles, std::max(per_group, 1)), (unsigned)groups), block(64 * nb);
#define JQ_QUADS(MAXNB)                                                                                            \
    hipLaunchKernelGGL((jq::moe_q4k_quads_mfma<MAXNB, DUAL>), grid, block, 0, s, Wa, Wb, xq, gexp, offsets, xsel,  \
                       yrow, Y, k, n, cl)
    if (maxnb == 16) JQ_QUADS(16);
    else if (maxnb == 8) JQ_QUADS(8);
    else JQ_QUADS(4);
#undef JQ_QUADS
    HIP_TRY(hipGetLastError());
    return 0;
}

// Lanes a row of moe_rows_dot8: 16, 32 or 64 by the row's units, so short rows fill the wave; 32 instead of 64
// where two rows make whole 16-byte pieces and one does not (IQ2_XXS rows of 7168: 1848 bytes), so that a wave's
// two rows go to LDS 16 bytes a lane and load instead of 4 (DeepSeek-V3 sizes, 8 tokens: 379 -> 339 us).
static int moe_dot8_lanes(int units, size_t row_bytes, int n, int base_align) {
    if (units < 48) return units >= 24 ? 32 : 16;
    return row_bytes % 16 != 0 && (2 * row_bytes) % 16 == 0 && n % 2 == 0 && base_align >= 16 ? 32 : 64;
}

// One activation row a group, a format with Q::dot8: expert rows staged through LDS and multiplied on
// v_dot4 against the activation row as int8 planes, quantised by every workgroup itself (small
// matrices) or once by acts_i8_prep (x_rows rows of X).  Returns -1 when the shape is outside its reach.
template <class Q, bool DUAL>
int launch_moe_dot8(const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align, const float *X,
                    size_t x_rows, jq::ActsI8 xq, const int *gexp, const int *offsets, const int *xsel, const int *yrow,
                    float *Y, int k, int n, int groups, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{},
                    bool planes_ready = false) {
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS;
    const int L = moe_dot8_lanes(units, row_bytes, n, base_align), R = 64 / L;
    const int G = (((size_t)R * row_bytes) % 16 == 0 && n % R == 0 && base_align >= 16) ? 16 : (row_bytes % 4 == 0 && base_align >= 4) ? 4 : 0;
    // every workgroup of a group redoing the row's quantisation is cheaper than a launch up to about
    // half a million elements a group (moe_dot8_takes_planes says the same)
    const size_t wgs = (n + jq::ROWS_PER_WG * R - 1) / (jq::ROWS_PER_WG * R);
    const bool own = wgs * (size_t)k <= 512 * 1024 || !xq.xl;
    const size_t one = ((size_t)R * row_bytes + 15) / 16 * 16, wave_lds = one * (DUAL ? 2 : 1);
    const size_t lds = wave_lds * jq::ROWS_PER_WG + jq::table_bytes<Q>() + (own ? (size_t)k * 2 + (size_t)k / 4 : 0);
    if (G == 0 || lds > 64 * 1024) return -1;
    if (!own && !planes_ready) {
        const size_t words = x_rows * (size_t)(k / 4);
        hipLaunchKernelGGL(jq::acts_i8_prep, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, X, x_rows, k, xq);
    }
    dim3 grid((unsigned)wgs, (unsigned)groups), block(64 * jq::ROWS_PER_WG);
#define JQ_DOT8(GG, OWN)                                                                                          \
    hipLaunchKernelGGL((jq::moe_rows_dot8<Q, DUAL, GG, OWN>), grid, block, lds, s, Wa, Wb, row_bytes, X, xq, gexp,  \
                       offsets, xsel, yrow, Y, k, n, L, (int)wave_lds, cl)
    if (G == 16 && own) JQ_DOT8(16, true);
    else if (G == 16) JQ_DOT8(16, false);
    else if (own) JQ_DOT8(4, true);
    else JQ_DOT8(4, false);
#undef JQ_DOT8
    note_kernel("moe_rows_dot8");
    HIP_TRY(hipGetLastError());
    return 0;
}

// Several pairs a group (bucketed by expert), a format with Q::decode_i8: moe_expert_dot8 over acts_i8_prep's
// planes of the x_rows rows of X.  Returns -1 when the shape is outside its reach.
template <class Q, bool DUAL>
int launch_moe_expert_dot8(const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align,
                           const float *X, size_t x_rows, jq::ActsI8 xq, const int *gexp, const int *offsets, const int *xsel,
                           const int *yrow, float *Y, int k, int n, int groups, hipStream_t s,
                           const jq::MoeClamp &cl = jq::MoeClamp{}) {
    const int units = k / 32;
    // lanes a row: the fewest of 16, 32, 64 that leave a lane at most seven units (eight for the longest rows)
    const int L = units <= 112 ? 16 : units <= 224 ? 32 : 64, R = 64 / L, ul = (units + L - 1) / L;
    constexpr size_t XB = 68 + (Q::I8_HAS_MIN ? 4 : 0);
    const size_t wgs = (n + jq::EXPERT_DOT8_WAVES * R - 1) / (jq::EXPERT_DOT8_WAVES * R);
    // a wave copies its R rows as one run of bytes: 16 bytes a lane when the run is whole pieces of 16 (IQ2_XXS rows
    // of 7168: 1848 bytes, two of them 231 pieces), else 4
    const int G = (((size_t)R * row_bytes) % 16 == 0 && n % R == 0 && base_align >= 16) ? 16
                  : (row_bytes % 4 == 0 && base_align >= 4)                              ? 4
                                                                                         : 0;
    const size_t one = ((size_t)R * row_bytes + 15) / 16 * 16, wave_lds = one * (DUAL ? 2 : 1);
    const size_t tables = jq::table_bytes<Q>() + 8 * Q::I8_EXTRA_ENTRIES, rows_lds = jq::EXPERT_DOT8_WAVES * wave_lds;
    // the activation buffers behind the rows when both fit, else in their place once the rows are decoded
    const size_t x_at = rows_lds + 2 * XB * units + tables <= 64 * 1024 ? rows_lds : 0;
    const size_t lds = std::max(rows_lds, x_at + 2 * XB * units) + tables;
    if (k % 128 != 0 || ul > 8 || G == 0 || lds > 64 * 1024 || !xq.xl) return -1;
    const size_t words = x_rows * (size_t)(k / 4);
    hipLaunchKernelGGL(jq::acts_i8_prep, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, X, x_rows, k, xq);
    dim3 grid((unsigned)wgs, (unsigned)groups), block(64 * jq::EXPERT_DOT8_WAVES);
#define JQ_EXPERT_DOT8(UL_)                                                                                         \
    case UL_:                                                                                                       \
        if (G == 16)                                                                                                \
            hipLaunchKernelGGL((jq::moe_expert_dot8<Q, DUAL, 16, UL_>), grid, block, lds, s, Wa, Wb, row_bytes, xq, gexp,  \
                               offsets, xsel, yrow, Y, k, n, L, (int)wave_lds, (int)x_at, cl);                      \
        else                                                                                                        \
            hipLaunchKernelGGL((jq::moe_expert_dot8<Q, DUAL, 4, UL_>), grid, block, lds, s, Wa, Wb, row_bytes, xq, gexp,   \
                               offsets, xsel, yrow, Y, k, n, L, (int)wave_lds, (int)x_at, cl);                      \
        break;
    switch (ul) {
        JQ_EXPERT_DOT8(1) JQ_EXPERT_DOT8(2) JQ_EXPERT_DOT8(3) JQ_EXPERT_DOT8(4)
        JQ_EXPERT_DOT8(5) JQ_EXPERT_DOT8(6) JQ_EXPERT_DOT8(7) JQ_EXPERT_DOT8(8)
    }
#undef JQ_EXPERT_DOT8
    note_kernel("moe_expert_dot8");
    HIP_TRY(hipGetLastError());
    return 0;
}

template <bool DUAL>
int dispatch_moe_expert_dot8(uint32_t type, const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes,
                             int base_align, const float *X, size_t x_rows, jq::ActsI8 xq, const int *gexp,
                             const int *offsets, const int *xsel, const int *yrow, float *Y, int k, int n, int groups,
                             hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    if (((uintptr_t)X & 15) != 0) return -1;
    switch (type) {
    case JQ_TYPE_MXFP4:
        return launch_moe_expert_dot8<jq::MXFP4, DUAL>(Wa, Wb, row_bytes, base_align, X, x_rows, xq, gexp, offsets, xsel, yrow,
                                                       Y, k, n, groups, s, cl);
    case JQ_TYPE_IQ2_XXS:
        return launch_moe_expert_dot8<jq::IQ2_XXS, DUAL>(Wa, Wb, row_bytes, base_align, X, x_rows, xq, gexp, offsets, xsel,
                                                         yrow, Y, k, n, groups, s, cl);
    case JQ_TYPE_Q4_K:
        return launch_moe_expert_dot8<jq::Q4_K, DUAL>(Wa, Wb, row_bytes, base_align, X, x_rows, xq, gexp, offsets, xsel, yrow,
                                                      Y, k, n, groups, s, cl);
    default: return -1;
    }
}

// Whether launch_moe_dot8 reads the activation planes acts_i8_prep makes (long rows) instead of quantising the row
// in every workgroup.
bool moe_dot8_takes_planes(uint32_t type, size_t row_bytes, int base_align, int k, int n, const jq::ActsI8 &xq) {
    if (!moe_has_dot8(type) || k % 32 != 0 || !xq.xl) return false;
    const int units = type == JQ_TYPE_Q4_K ? k / 64 : k / 32;
    const int R = 64 / moe_dot8_lanes(units, row_bytes, n, base_align);
    const size_t wgs = (n + jq::ROWS_PER_WG * R - 1) / (jq::ROWS_PER_WG * R);
    return wgs * (size_t)k > 512 * 1024;
}

template <bool DUAL>
int dispatch_moe_dot8(uint32_t type, const uint8_t *const *Wa, const uint8_t *const *Wb, size_t row_bytes, int base_align,
                      const float *X, size_t x_rows, jq::ActsI8 xq, const int *gexp, const int *offsets,
                      const int *xsel, const int *yrow, float *Y, int k, int n, int groups, hipStream_t s,
                      const jq::MoeClamp &cl = jq::MoeClamp{}, bool planes_ready = false) {
    if (!moe_has_dot8(type) || k % 32 != 0 || ((uintptr_t)X & 15) != 0) return -1;
    switch (type) {
#define JQ_DOT8_CASE(ID, Q)                                                                                         \
    case ID:                                                                                                        \
        return launch_moe_dot8<jq::Q, DUAL>(Wa, Wb, row_bytes, base_align, X, x_rows, xq, gexp, offsets, xsel, yrow, Y, k, n, \
                                            groups, s, cl, planes_ready);
        JQ_DOT8_CASE(JQ_TYPE_MXFP4, MXFP4)
        JQ_DOT8_CASE(JQ_TYPE_IQ2_XXS, IQ2_XXS)
        JQ_DOT8_CASE(JQ_TYPE_Q4_K, Q4_K)
#undef JQ_DOT8_CASE
    default: return -1;
    }
}

// The decode-sized down projection and the weighted combine in one launch (moe_down_combine_dot8): T
// tokens, k_used routed pairs each plus n_extra for a folded shared expert, activations the rows of X
// in pair order.  Returns -1 when the shape is outside its reach.
template <class Q>
int launch_moe_down_combine(const uint8_t *const *Wa, size_t row_bytes, int base_align, const float *X, size_t x_rows,
                            jq::ActsI8 xq, const int *gexp, const float *wts, float *y, int k, int n, int T, int k_used,
                            int n_extra, hipStream_t s) {
    const int units = (k / Q::BLOCK_ELEMS) * Q::UNITS, S = k_used + n_extra;
    const int L = units >= 48 ? 64 : units >= 24 ? 32 : 16, R = 64 / L;
    const int G = (row_bytes % 16 == 0 && base_align >= 16) ? 16 : (row_bytes % 4 == 0 && base_align >= 4) ? 4 : 0;
    const size_t wgs = (n + jq::ROWS_PER_WG * R - 1) / (jq::ROWS_PER_WG * R);
    const bool own = wgs * (size_t)k <= 512 * 1024 || !xq.xl;  // as in launch_moe_dot8
    const size_t slot_lds = ((size_t)R * row_bytes + 15) / 16 * 16;
    const size_t lds = slot_lds * S * jq::ROWS_PER_WG + jq::table_bytes<Q>() + (own ? (size_t)S * ((size_t)k * 2 + (size_t)k / 4) : 0);
    // worth it from two workgroups a compute unit on: each one works through its S pairs in turn
    if (G == 0 || S > 64 || lds > 96 * 1024 || T > 65535 || k % 16 != 0 || wgs * (size_t)T < 512) return -1;
    if (!own) {
        const size_t words = x_rows * (size_t)(k / 4);
        hipLaunchKernelGGL(jq::acts_i8_prep, dim3((unsigned)((words + 255) / 256)), dim3(256), 0, s, X, x_rows, k, xq);
    }
    dim3 grid((unsigned)wgs, (unsigned)T), block(64 * jq::ROWS_PER_WG);
#define JQ_DC(GG, OWN)                                                                                              \
    do {                                                                                                            \
        auto kern = jq::moe_down_combine_dot8<Q, GG, OWN>;                                                          \
        static std::once_flag big_lds;                                                                              \
        static hipError_t attr_rc = hipSuccess;                                                                     \
        std::call_once(big_lds, [&] {                                                                               \
            attr_rc = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024); \
        });                                                                                                         \
        HIP_TRY(attr_rc);                                                                                           \
        hipLaunchKernelGGL(kern, grid, block, lds, s, Wa, row_bytes, X, xq, gexp, wts, y, k, n, L, (int)slot_lds,  \
                           k_used, n_extra, T * k_used);                                                            \
    } while (0)
    if (G == 16 && own) JQ_DC(16, true);
    else if (G == 16) JQ_DC(16, false);
    else if (own) JQ_DC(4, true);
    else JQ_DC(4, false);
#undef JQ_DC
    note_kernel("moe_down_combine_dot8");
    HIP_TRY(hipGetLastError());
    return 0;
}

int dispatch_moe_down_combine(uint32_t type, const uint8_t *const *Wa, size_t row_bytes, int base_align, const float *X,
                              size_t x_rows, jq::ActsI8 xq, const int *gexp, const float *wts, float *y, int k, int n,
                              int T, int k_used, int n_extra, hipStream_t s) {
    static const char *off = getenv("JQ_MOE_NO_DOWN_COMBINE");
    if (off || !moe_has_dot8(type) || k % 32 != 0 || ((uintptr_t)X & 15) != 0) return -1;
    switch (type) {
#define JQ_DC_CASE(ID, Q)                                                                                           \
    case ID:                                                                                                        \
        return launch_moe_down_combine<jq::Q>(Wa, row_bytes, base_align, X, x_rows, xq, gexp, wts, y, k, n, T, k_used, \
                                              n_extra, s);
        JQ_DC_CASE(JQ_TYPE_MXFP4, MXFP4)
        JQ_DC_CASE(JQ_TYPE_IQ2_XXS, IQ2_XXS)
        JQ_DC_CASE(JQ_TYPE_Q4_K, Q4_K)
#undef JQ_DC_CASE
    default: return -1;
    }
}

// The decode-sized expert matmuls on the int8 matrix cores (kernels_moe_mfma.hpp).  -1: outside their reach
// (format without a policy, rows that are not 1, 2, 4 or 8 super-blocks for gate and up or more than 16 for down,
// rows that do not start on 16 bytes).
template <class K>
int moe_mfma_big_lds(K kern, int lds) {
    if (lds <= 64 * 1024) return 0;
    HIP_TRY(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds));
    return 0;
}

jq::MoeStack moe_stack(const jq_weight *w, size_t rows_per_expert, size_t n_expert, const jq_weight *extra) {
    return jq::MoeStack{w->dev, rows_per_expert * w->row_bytes, extra ? extra->dev : w->dev, (int)n_expert};
}

// Bytes of a 256-element super-block in the formats the matrix-core expert kernels have a policy for; 0: none.
int moe_mfma_block_bytes(uint32_t type) {
    switch (type) {
    case JQ_TYPE_Q4_K: return jq::QvQ4K::BLOCK;
    case JQ_TYPE_IQ2_XXS: return jq::QvI8<jq::IQ2_XXS>::BLOCK;
    case JQ_TYPE_MXFP4: return jq::QvI8<jq::MXFP4>::BLOCK;
    default: return 0;
    }
}

// Does a matrix-core kernel take this layer's gate and up projections?  Rows of 1, 2, 4 or 8 super-blocks (Q4_K;
// 8 for the others): moe_gate_up_mfma; of 9 to 32: moe_gate_up_rows_mfma.
bool moe_gate_up_mfma_takes(const jq_moe *m, const float *X) {
    static const char *off = getenv("JQ_MOE_NO_MFMA");
    const jq_moe_config &c = m->cfg;
    const int nb = (int)(c.hidden / 256), bb = moe_mfma_block_bytes(m->gate->type);
    if (off || !bb || m->up->type != m->gate->type || c.hidden % 256 != 0 || ((uintptr_t)X & 15) != 0) return false;
    if (m->gate->row_bytes != (size_t)nb * bb || m->up->row_bytes != m->gate->row_bytes) return false;
    uintptr_t bits = (uintptr_t)m->gate->dev | (uintptr_t)m->up->dev;
    if (m->fold_shared) bits |= (uintptr_t)m->sgate->dev | (uintptr_t)m->sup->dev;
    if ((bits & 15) != 0) return false;
    // JQ_MOE_MFMA_ONLY=gate_up / down: only that projection takes the matrix-core kernels (for measurements)
    static const char *only = getenv("JQ_MOE_MFMA_ONLY");
    const char only_part = only ? only[0] : 0;
    if (only_part == 'd') return false;
    if (nb <= 8) return nb == 8 || (m->gate->type == JQ_TYPE_Q4_K && (nb == 1 || nb == 2 || nb == 4));
    // whole rows of a tile as two spans of 8 rows, copied by 1024 lanes in one instruction (IQ2_XXS) or two, through a
    // ring of two slots; the slot behind the first holds the waves' raw activations (1 KB a column) at the start
    const bool iq2 = m->gate->type == JQ_TYPE_IQ2_XXS;
    const size_t pieces = (size_t)nb * bb / 2, slot = (size_t)16 * nb * bb;
    const size_t lds = iq2 ? jq::moe_gate_up_rows_mfma_lds<jq::QvI8<jq::IQ2_XXS>, 2, 2, 1>(nb)
                           : m->gate->type == JQ_TYPE_MXFP4 ? jq::moe_gate_up_rows_mfma_lds<jq::QvI8<jq::MXFP4>, 2, 2, 2>(nb)
                                                            : jq::moe_gate_up_rows_mfma_lds<jq::QvQ4K, 2, 2, 2>(nb);
    return nb <= 32 && c.inter % 8 == 0 && pieces <= (iq2 ? 1024u : 2048u) && slot >= (size_t)nb * 1024 && lds <= 158 * 1024;
}

// MXFP4 and Q4_K rows that are whole 16-byte pieces of at most 4 KB travel row by row into padded LDS rows
// (JQ_MOE_GATE_UP_SPANS: as spans of 8 rows like the other shapes).
template <class F>
bool moe_gate_up_rows_padded(int nb) {
    static const char *spans = getenv("JQ_MOE_GATE_UP_SPANS");
    const int rb = nb * F::BLOCK;
    return !spans && rb % 16 == 0 && rb <= 4096 && jq::moe_gate_up_rows_mfma_lds<F, 2, 2, 2, true>(nb) <= 158 * 1024;
}

// `gate`: the launch runs the gating of the T tokens too (the router's logits are in m->logits).
int dispatch_moe_gate_up_mfma(const jq_moe *m, const float *X, int pairs, hipStream_t s, const jq::MoeClamp &cl, float *zero,
                              int zero_n, const jq::MoeGateIn *gate) {
    const jq_moe_config &c = m->cfg;
    if (!moe_gate_up_mfma_takes(m, X) || pairs <= 0 || pairs > 65535) return -1;
    const int nb = (int)(c.hidden / 256), n = (int)c.inter;
    const jq::MoeStack wa = moe_stack(m->gate, c.inter, c.n_expert, m->fold_shared ? m->sgate : nullptr),
                       wb = moe_stack(m->up, c.inter, c.n_expert, m->fold_shared ? m->sup : nullptr);
    const jq::MoeGateIn gi = gate ? *gate : jq::MoeGateIn{};
#define JQ_GU(F, NB, GATE)                                                                                            \
    do {                                                                                                              \
        auto kern = jq::moe_gate_up_mfma<F, NB, GATE>;                                                                \
        constexpr int lds = jq::moe_gate_up_mfma_lds<F, NB>();                                                        \
        static const int attr_rc = moe_mfma_big_lds(kern, lds);                                                       \
        if (attr_rc) return 1;                                                                                        \
        hipLaunchKernelGGL(kern, dim3((unsigned)((n + 7) / 8), (unsigned)pairs), dim3(64 * NB), lds, s, wa, wb, X, m->gexp, \
                           m->xrow, m->yrow, m->G, n, cl, zero, zero_n, gi);                                          \
    } while (0)
    // rows of more than 8 super-blocks: 16 waves a pair and tile sequence, two columns a wave
#define JQ_GUR(F, SL, J, GATE) JQ_GUR_(F, SL, J, GATE, false)
#define JQ_GUR_(F, SL, J, GATE, ROWS)                                                                                 \
    do {                                                                                                              \
        auto kern = jq::moe_gate_up_rows_mfma<F, 2, SL, J, GATE, ROWS>;                                               \
        const int lds = jq::moe_gate_up_rows_mfma_lds<F, 2, SL, J, ROWS>(nb);                                         \
        const int slot = jq::moe_gate_up_rows_slot<F, ROWS>(nb);                                                      \
        if (lds > 158 * 1024 || (SL - 1) * slot < nb * 1024 || zero) return -1;                                   \
        static const int attr_rc = moe_mfma_big_lds(kern, 158 * 1024);                                                \
        if (attr_rc) return 1;                                                                                        \
        const int per_pair = std::max(1, std::min(n / 8, (lds > 79 * 1024 ? 256 : 512) / pairs));                     \
        hipLaunchKernelGGL(kern, dim3((unsigned)per_pair, (unsigned)pairs), dim3(1024), lds, s, wa, wb, X, m->gexp, m->xrow, \
                           m->yrow, m->G, n, nb, cl, gi);                                                             \
    } while (0)
    const uint32_t type = m->gate->type;
    if (nb > 8) {
        if (type == JQ_TYPE_IQ2_XXS && gate) JQ_GUR(jq::QvI8<jq::IQ2_XXS>, 2, 1, true);
        else if (type == JQ_TYPE_IQ2_XXS) JQ_GUR(jq::QvI8<jq::IQ2_XXS>, 2, 1, false);
        else if (type == JQ_TYPE_MXFP4 && moe_gate_up_rows_padded<jq::QvI8<jq::MXFP4>>(nb) && gate) JQ_GUR_(jq::QvI8<jq::MXFP4>, 2, 2, true, true);
        else if (type == JQ_TYPE_MXFP4 && moe_gate_up_rows_padded<jq::QvI8<jq::MXFP4>>(nb)) JQ_GUR_(jq::QvI8<jq::MXFP4>, 2, 2, false, true);
        else if (type == JQ_TYPE_MXFP4 && gate) JQ_GUR(jq::QvI8<jq::MXFP4>, 2, 2, true);
        else if (type == JQ_TYPE_MXFP4) JQ_GUR(jq::QvI8<jq::MXFP4>, 2, 2, false);
        else if (moe_gate_up_rows_padded<jq::QvQ4K>(nb) && gate) JQ_GUR_(jq::QvQ4K, 2, 2, true, true);
        else if (moe_gate_up_rows_padded<jq::QvQ4K>(nb)) JQ_GUR_(jq::QvQ4K, 2, 2, false, true);
        else if (gate) JQ_GUR(jq::QvQ4K, 2, 2, true);
        else JQ_GUR(jq::QvQ4K, 2, 2, false);
        note_kernel(gate ? "moe_gate_up_rows_mfma+gating" : "moe_gate_up_rows_mfma");
        HIP_TRY(hipGetLastError());
        return 0;
    }
    if (type == JQ_TYPE_IQ2_XXS && gate) JQ_GU(jq::QvI8<jq::IQ2_XXS>, 8, true);
    else if (type == JQ_TYPE_IQ2_XXS) JQ_GU(jq::QvI8<jq::IQ2_XXS>, 8, false);
    else if (type == JQ_TYPE_MXFP4 && gate) JQ_GU(jq::QvI8<jq::MXFP4>, 8, true);
    else if (type == JQ_TYPE_MXFP4) JQ_GU(jq::QvI8<jq::MXFP4>, 8, false);
    else if (nb == 8 && gate) JQ_GU(jq::QvQ4K, 8, true);
    else if (nb == 8) JQ_GU(jq::QvQ4K, 8, false);
    else if (nb == 4 && gate) JQ_GU(jq::QvQ4K, 4, true);
    else if (nb == 4) JQ_GU(jq::QvQ4K, 4, false);
    else if (nb == 2 && gate) JQ_GU(jq::QvQ4K, 2, true);
    else if (nb == 2) JQ_GU(jq::QvQ4K, 2, false);
    else if (gate) JQ_GU(jq::QvQ4K, 1, true);
    else JQ_GU(jq::QvQ4K, 1, false);
#undef JQ_GU
#undef JQ_GUR
#undef JQ_GUR_
    note_kernel(gate ? "moe_gate_up_mfma+gating" : "moe_gate_up_mfma");
    HIP_TRY(hipGetLastError());
    return 0;
}

// `split`: the caller has cleared y and two workgroups may share a row tile.
int dispatch_moe_down_mfma(const jq_moe *m, const float *A, float *y, int T, int n_extra, bool split, hipStream_t s) {
    static const char *off = getenv("JQ_MOE_NO_MFMA");
    const jq_moe_config &c = m->cfg;
    const int k = (int)c.inter, n = (int)c.hidden, k_used = (int)c.n_expert_used, S = k_used + n_extra;
    const uint32_t type = m->down->type;
    // (Q6_K: rows of three 210-byte blocks, the down projections of a Q4_K_M file's layers with more bits)
    const int bb = type == JQ_TYPE_Q6_K ? jq::QvQ6K::BLOCK : moe_mfma_block_bytes(type);
    uintptr_t bits = (uintptr_t)m->down->dev | (uintptr_t)A;
    if (m->fold_shared) bits |= (uintptr_t)m->sdown->dev;
    static const char *only = getenv("JQ_MOE_MFMA_ONLY");
    if (off || (only && only[0] == 'g') || !bb || k % 256 != 0 || (bits & 15) != 0 || S > 64 || T <= 0 || T > 65535) return -1;
    const int nb = k / 256;
    if (m->down->row_bytes != (size_t)nb * bb || nb > 16) return -1;
    if (type == JQ_TYPE_Q6_K ? (nb != 3 || n % 16 != 0) : (type != JQ_TYPE_Q4_K && nb != 8)) return -1;
    const jq::MoeStack wd = moe_stack(m->down, c.hidden, c.n_expert, m->fold_shared ? m->sdown : nullptr);
#define JQ_DN(F, NB, SPP, SL, XB, ...)                                                                                       \
    do {                                                                                                              \
        auto kern = jq::moe_down_mfma<F, NB, SPP, SL, XB, ##__VA_ARGS__>;                                                            \
        constexpr int lds = jq::moe_down_mfma_lds<F, NB, SPP, SL, XB, ##__VA_ARGS__>();                                              \
        static_assert(lds <= 158 * 1024, "the ring fits a compute unit");                                             \
        static const int attr_rc = moe_mfma_big_lds(kern, lds);                                                       \
        if (attr_rc) return 1;                                                                                        \
        const unsigned z = split && (S + SPP - 1) / SPP == 2 ? 2 : 1;                                                 \
        if (split && z == 1) return -1;                                                                               \
        hipLaunchKernelGGL(kern, dim3((unsigned)((n + 15) / 16), (unsigned)T, z), dim3(1024), lds, s, wd, A, m->gexp, m->wts, \
                           y, n, k_used, n_extra, T * k_used);                                                        \
    } while (0)
    // segments a pass: as many as fill the 16 waves, or fewer when the passes then come out even
    // (IQ2_XXS: two slots and one activation buffer, 74 KB, two workgroups a compute unit)
    if (type == JQ_TYPE_IQ2_XXS) JQ_DN(jq::QvI8<jq::IQ2_XXS>, 8, 2, 2, 1);
    else if (type == JQ_TYPE_MXFP4) JQ_DN(jq::QvI8<jq::MXFP4>, 8, 2, 2, 2);
    else if (type == JQ_TYPE_Q6_K && (S + 3) / 4 == (S + 4) / 5) JQ_DN(jq::QvQ6K, 3, 4, 2, 1, true);
    else if (type == JQ_TYPE_Q6_K) JQ_DN(jq::QvQ6K, 3, 5, 2, 1, true);
    else if (nb == 3 && (S + 3) / 4 == (S + 4) / 5) JQ_DN(jq::QvQ4K, 3, 4, 3, 2);
    else if (nb == 3) JQ_DN(jq::QvQ4K, 3, 5, 2, 2);
    else if (nb == 8) JQ_DN(jq::QvQ4K, 8, 2, 2, 2);
    else if (nb == 4) JQ_DN(jq::QvQ4K, 4, 4, 2, 2);
    else if (nb == 2) JQ_DN(jq::QvQ4K, 2, 8, 2, 2);
    else if (nb == 1) JQ_DN(jq::QvQ4K, 1, 16, 2, 2);
    else return -1;
#undef JQ_DN
    note_kernel("moe_down_mfma");
    HIP_TRY(hipGetLastError());
    return 0;
}

// Would dispatch_moe_down_mfma run this call with two workgroups a row tile (into a cleared y)?
bool moe_down_mfma_splits(const jq_moe *m, int T, int n_extra) {
    const jq_moe_config &c = m->cfg;
    const int S = (int)c.n_expert_used + n_extra, nb = (int)(c.inter / 256);
    if (c.inter % 256 != 0 || nb < 1 || nb > 16 || (nb > 4 && nb != 8)) return false;
    const int spp = nb == 3 ? ((S + 3) / 4 == (S + 4) / 5 ? 4 : 5) : 16 / nb;
    return (S + spp - 1) / spp == 2 && (size_t)T * ((c.hidden + 15) / 16) <= 128;
}

template <bool SWIGLU>
int dispatch_moe_rows(uint32_t type, const uint8_t *const *Wptr, size_t row_bytes, const float *X, const float *X2,
                      const int *gexp, const int *offsets, const int *xsel, const int *yrow, float *Y, int k, int n,
                      int groups, int max_group, hipStream_t s, const jq::MoeClamp &cl = jq::MoeClamp{}) {
    switch (type) {
#define JQ_MOE_CASE(ID, Q)                                                                                          \
    case ID:                                                                                                        \
        launch_moe_rows<jq::Q, SWIGLU>(Wptr, row_bytes, X, X2, gexp, offsets, xsel, yrow, Y, k, n, groups, max_group, \
                                       s, cl);                                                                      \
        break;
        JQ_FOR_EACH_FORMAT(JQ_MOE_CASE)
#undef JQ_MOE_CASE
    default: return fail("unsupported tensor type id %u", type);
    }
    HIP_TRY(hipGetLastError());
    return 0;
}

// One grouped expert matmul on the int8 GEMM: activation rows X[xsel[pair]] prepared into m->gacts (unless
// `prepared`: the previous call left the same ones there) by the tables in m->gtab, results to Y[m->yrow[pair]].
// Returns -1 when the matrix is outside its reach.
jq::QiGroupTables moe_gemm_tables(const jq_moe *m) {
    const size_t R = m->gtab_rows;
    return jq::QiGroupTables{m->gtab, m->gtab + R, m->gtab + 2 * R, m->gtab + 3 * R, m->gtab + 4 * R, m->gtab + 8 * R};
}
// (the mixed plan's tiles of two row groups; their count sits where a launch looks for it: at counts[1])
jq::QiGroupTables moe_gemm_tables_small(const jq_moe *m) {
    const size_t R = m->gtab_rows;
    return jq::QiGroupTables{m->gtab, m->gtab + R, m->gtab + 5 * R, m->gtab + 6 * R, m->gtab + 7 * R, m->gtab + 8 * R + 1};
}

template <class F>
int launch_moe_gemm_i8(jq_moe *m, const uint8_t *const *wptr, size_t row_bytes, int base_align, const float *X,
                       const int *xsel, bool prepared, float *Y, int k, int n, hipStream_t s) {
    if (!m->gacts || k % 256 != 0 || row_bytes % F::ALIGN != 0 || base_align < F::ALIGN) return -1;
    constexpr int NG = 4;
    const size_t nb = (size_t)k / 256, tx = ((size_t)n + 16 * NG - 1) / (16 * NG);
    const size_t max_rg = m->gtab_rows;
    if (tx * max_rg > 0x7FFFFFFFull) return -1;
    const jq::QiGroupTables t = moe_gemm_tables(m);
    if (!prepared)
        hipLaunchKernelGGL((jq::moe_gemm_i8_prep<F::SUB16>), dim3((unsigned)nb, (unsigned)max_rg), dim3(256), 0, s, X, xsel, t, k,
                           m->gacts);
    hipError_t attr_rc = hipSuccess;
    // (the tiles of few rows on one operand buffer: four workgroups a compute unit instead of two.  JQ_MOE_GEMM_DOUBLE_BUFFER
    // keeps the two buffers)
    static const char *double_env = getenv("JQ_MOE_GEMM_DOUBLE_BUFFER");
    // most tiles a plan can hold: every tile of the mixed plan's first list has five row groups or more, its second
    // list at most two tiles an expert
    const size_t n_groups = m->cfg.n_expert + (m->fold_shared ? 1 : 0);
    const size_t max_big = m->gtile_rgs == 0 ? max_rg / 5 + 1 : max_rg, max_small = m->gtile_rgs == 0 ? 2 * n_groups : max_rg;
#define JQ_MOE_GEMM(NW_, NSPLIT_) JQ_MOE_GEMM_(NW_, NSPLIT_, false)
#define JQ_MOE_GEMM_(NW_, NSPLIT_, SINGLE_)                                                                           \
    do {                                                                                                              \
        auto kern = jq::kq_gemm_i8<F, NW_, NG, true, NSPLIT_, SINGLE_>;                                               \
        constexpr int lds = jq::qi_lds_bytes<F, NG, SINGLE_>();                                                       \
        static std::once_flag big_lds;                                                                                \
        static hipError_t rc_once = hipSuccess;                                                                       \
        std::call_once(big_lds, [&] {                                                                                 \
            rc_once = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);       \
        });                                                                                                           \
        attr_rc = rc_once;                                                                                            \
        const jq::QiGrouped gp{wptr, m->gexp, m->yrow, NSPLIT_ && m->gtile_rgs == 0 ? moe_gemm_tables_small(m) : t};   \
        const size_t max_mt = NSPLIT_ ? max_small : max_big;                                                          \
        if (attr_rc == hipSuccess)                                                                                    \
            hipLaunchKernelGGL(kern, dim3((unsigned)(tx * max_mt)), dim3(64 * NW_), lds, s, (const uint8_t *)nullptr, \
                               row_bytes, (const uint8_t *)m->gacts, Y, 0, n, (int)nb, 0, (int)tx, 0, (int)nb,       \
                               (size_t)0, gp);                                                                        \
    } while (0)
    if (m->gtile_rgs != 2) JQ_MOE_GEMM(4, false);
    if (m->gtile_rgs != 8 && attr_rc == hipSuccess) {
        if (double_env) JQ_MOE_GEMM(2, true);
        else JQ_MOE_GEMM_(2, true, true);
    }
#undef JQ_MOE_GEMM
#undef JQ_MOE_GEMM_
    HIP_TRY(attr_rc);
    note_kernel(m->gtile_rgs == 2 ? "moe_gemm_i8_few" : m->gtile_rgs == 0 ? "moe_gemm_i8_mixed" : "moe_gemm_i8");
    HIP_TRY(hipGetLastError());
    return 0;
}

// The tile plan of a bucketed call: few pairs an expert (32 on average or fewer) -> tiles of two row groups whose
// waves share the weight rows; more -> tiles of eight row groups whose waves share the rows.
void moe_gemm_plan(jq_moe *m, int groups, size_t pairs, hipStream_t s) {
    // Few pairs an expert on average (under 8): every tile two row groups.  More: the mixed plan, since the pairs of a
    // call are seldom spread evenly (a prompt of one repeated token sends all its pairs to eight experts) and the
    // host does not know how they fell: eight row groups a tile where an expert has them, two for the rest.
    static const char *env = getenv("JQ_MOE_GEMM_TILE_ROWS");  // 32 or 128: that tile for every call; 0: the mixed plan
    m->gtile_rgs = env ? (atoi(env) == 32 ? 2 : atoi(env) == 128 ? 8 : 0) : (pairs < 8 * (size_t)groups ? 2 : 0);
    hipLaunchKernelGGL(jq::moe_gemm_i8_plan, dim3(1), dim3(256), 0, s, m->offsets, groups, m->gtile_rgs, moe_gemm_tables(m),
                       moe_gemm_tables_small(m));
}

int dispatch_moe_gemm_i8(jq_moe *m, uint32_t type, const uint8_t *const *wptr, size_t row_bytes, int base_align,
                         const float *X, const int *xsel, bool prepared, float *Y, int k, int n, hipStream_t s) {
    if (!moe_has_gemm_i8(type)) return -1;
    switch (type) {
#define JQ_QI_CASE(ID, F) \
    case ID: return launch_moe_gemm_i8<jq::F>(m, wptr, row_bytes, base_align, X, xsel, prepared, Y, k, n, s);
        JQ_QI_CASE(JQ_TYPE_Q4_K, QiQ4K)
        JQ_QI_CASE(JQ_TYPE_Q6_K, QiQ6K)
        JQ_QI_CASE(JQ_TYPE_Q2_K, QiQ2K)
        JQ_QI_CASE(JQ_TYPE_Q8_0, QiQ8_0)
        JQ_QI_CASE(JQ_TYPE_IQ2_XXS, QiIQ2XXS)
        JQ_QI_CASE(JQ_TYPE_MXFP4, QiMXFP4)
        JQ_QI_CASE(JQ_TYPE_Q5_K, QiQ5K)
        JQ_QI_CASE(JQ_TYPE_Q4_0, QiQ4_0)
        JQ_QI_CASE(JQ_TYPE_Q3_K, QiQ3K)
        JQ_QI_CASE(JQ_TYPE_Q5_0, QiQ5_0)
        JQ_QI_CASE(JQ_TYPE_Q4_1, QiQ4_1)
        JQ_QI_CASE(JQ_TYPE_Q5_1, QiQ5_1)
#undef JQ_QI_CASE
    default: return -1;
    }
}

// `planes`: also leave x as fixed-point planes there (the one-expert-a-workgroup router kernel does; *planes_made
// says whether it ran)
// `gate_later`: when the gating can run by one wave a token, it is left to the caller's next kernel (the logits are
// in m->logits) and *gate_later holds its operands; else it is cleared.
// `pre`: the decoder layer's residual add and RMSNorm run inside the router launch (one token; x is then pre->hn_out,
// which that launch writes).
int moe_route_dev(jq_moe *m, size_t T, const float *x, hipStream_t s, jq::MoePairGroups pg,
                  jq::ActsI8 planes = jq::ActsI8{nullptr, nullptr, nullptr, nullptr}, bool *planes_made = nullptr,
                  jq::MoeGateIn *gate_later = nullptr, const jq::MoePreNormArgs *pre = nullptr) {
    const jq_moe_config &c = m->cfg;
    const unsigned token_runs = (unsigned)((T + jq::ROUTER_TOKENS_PER_WG - 1) / jq::ROUTER_TOKENS_PER_WG);
    static const char *no_tile = getenv("JQ_MOE_NO_ROUTER_TILE");
    // (a router of a million weights or more, 256 experts of 7168: from 8 tokens, 16 us against 27)
    const size_t tile_from = (size_t)c.hidden * c.n_expert >= (1u << 20) ? 8 : 32;
    jq::MoeGateParams gp{(int)c.n_expert, (int)c.n_expert_used, (int)c.gating, (int)c.norm_topk, c.weights_scale,
                         (int)c.n_group, (int)c.topk_group};
    static const char *no_wave = getenv("JQ_MOE_NO_WAVE_GATE");
    const bool wave_gate = !no_wave && c.n_group <= 1 && c.n_expert <= 256 && c.n_expert_used <= 64;
    if (pre)
        hipLaunchKernelGGL(jq::moe_router_logits_norm, dim3(c.n_expert), dim3(256), 0, s, m->router_w, *pre, m->logits,
                           (int)c.hidden, (int)c.n_expert);
    else if (T >= tile_from && !no_tile)  // many tokens: a token's activations read once per eight experts (the same bits)
        hipLaunchKernelGGL(jq::moe_router_logits_tile, dim3((c.n_expert + 7) / 8, (unsigned)((T + 7) / 8)), dim3(256), 0, s,
                           m->router_w, x, m->logits, (int)T, (int)c.hidden, (int)c.n_expert,
                           c.hidden % 32 == 0 ? planes : jq::ActsI8{nullptr, nullptr, nullptr, nullptr});
    else
        hipLaunchKernelGGL(jq::moe_router_logits, dim3(c.n_expert, token_runs), dim3(256), 0, s, m->router_w, x, m->logits,
                           (int)T, (int)c.hidden, (int)c.n_expert, planes);
    if (planes_made) *planes_made = !pre && planes.xl && (c.hidden % 32 == 0 || !(T >= tile_from && !no_tile));
    size_t sm = (2 * c.n_expert + std::max<uint32_t>(c.n_group, 1) + c.n_expert_used + 4) * sizeof(float);
    if (gate_later) {
        if (wave_gate) {
            *gate_later = jq::MoeGateIn{m->logits, m->router_bias, gp, m->ids, m->wts, pg, (int)T};
            HIP_TRY(hipGetLastError());
            return 0;
        }
        gate_later->logits = nullptr;
    }
    // no expert groups and at most 256 experts: one wave a token, reductions in registers
    if (wave_gate) {
        const int ne = (int)(c.n_expert + 63) / 64;
#define JQ_GATE(NE) hipLaunchKernelGGL(jq::moe_gate_topk_wave<NE>, dim3((unsigned)T), dim3(64), 0, s, m->logits, m->router_bias, gp, m->ids, m->wts, pg)
        if (ne == 1) JQ_GATE(1);
        else if (ne == 2) JQ_GATE(2);
        else if (ne == 3) JQ_GATE(3);
        else JQ_GATE(4);
#undef JQ_GATE
        HIP_TRY(hipGetLastError());
        return 0;
    }
    hipLaunchKernelGGL(jq::moe_gate_topk, dim3((unsigned)T), dim3(256), sm, s, m->logits, m->router_bias, gp, m->ids,
                       m->wts, pg);
    HIP_TRY(hipGetLastError());
    return 0;
}

// The decoder's residual add and RMSNorm in front of a layer's mixture of experts: x_out = x + res,
// hn_out = rmsnorm(x_out) w, and the experts run over hn_out.  `fused` says whether the router launch did it
// (then the caller's residual row is x_out) or a launch of its own in place (then it is still x).
struct MoePreNorm {
    jq::MoePreNormArgs a;
    bool fused;
};

int moe_forward_dev(jq_moe *m, size_t T, const float *x, float *y, hipStream_t s, MoePreNorm *pre = nullptr) {
    const jq_moe_config &c = m->cfg;
    const int P = (int)(T * c.n_expert_used), extra = m->fold_shared ? 1 : 0;
    // the experts' SwiGLU clamp; a folded shared expert is expert number n_expert and has its own
    const jq::MoeClamp clamp{c.swiglu_clamp, c.swiglu_clamp_shared, (int)c.n_expert};
    int groups, max_group;
    // Decode-sized (one group a pair, every pair reading its expert's rows) or bucketed by expert (every expert hit
    // read once)?  A pair costs about a = 0.10 + 0.17 bytes-per-weight ns a weight on the integer-dot kernels;
    // a bucketed expert costs g = 0.30 ns a weight on the grouped int8 GEMM (bound by the unpacking; 0.36 for Q4_K)
    // and 0.28 on the Q4_K kernels for short rows.  With d(P) = E (1 - (1 - 1/E)^P) experts hit by P pairs, pairs win
    // while P a <= d(P) g (Qwen3-30B-A3B sizes: up to ~100 pairs over 128 experts).  Formats without integer-dot
    // kernels keep pairs up to the number of experts.
    // MXFP4, IQ2_XXS and Q4_K have a third way, bucketed with the expert's rows decoded once into registers and the pairs
    // streamed past them (moe_expert_dot8): x = 0.10 ns a weight and expert hit plus 0.032 a pair, and about 90 us a
    // call for its launches over every (expert, row tile), most of them empty when few experts are hit.  At
    // DeepSeek-V3's sizes it is the cheapest from ~10 tokens (16 tokens of IQ2_XXS: 0.73 ms against 0.89 by pairs;
    // 64: 1.76 against 3.15; 256: 4.33 against the GEMM's 5.09) to ~350 (Q4_K: ~250), where the GEMM takes over.
    // JQ_MOE_DECODE_PAIRS_PCT: pairs, in percent of the experts, up to which a call is decode-sized.
    // JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT: bucketed calls take moe_expert_dot8 up to this many pairs an expert
    // on average (0: never).
    static const char *pct_env = getenv("JQ_MOE_DECODE_PAIRS_PCT");
    const char *expert_env = getenv("JQ_MOE_EXPERT_DOT8_UPTO_PAIRS_PER_EXPERT");  // read at every call
    const bool has_expert_dot8 = moe_has_decode_i8(m->gate->type) && m->gate->type == m->up->type &&
                                 moe_has_decode_i8(m->down->type) && c.hidden % 128 == 0 && c.inter % 128 == 0 && m->qi8.xl;
    bool decode_sized = (size_t)P <= c.n_expert;
    bool expert_dot8 = expert_env && has_expert_dot8 && (size_t)P <= (size_t)atoll(expert_env) * c.n_expert;
    if (pct_env) {
        decode_sized = (size_t)P * 100 <= c.n_expert * (size_t)atoll(pct_env);
    } else if (expert_dot8) {
        // asked for: every call of more pairs than experts, up to the given number an expert
    } else if (moe_has_dot8(m->gate->type) && moe_has_dot8(m->up->type) && moe_has_dot8(m->down->type) &&
               c.hidden % 256 == 0 && c.inter % 256 == 0) {
        const double bpw = (double)m->gate->row_bytes / (double)c.hidden;
        const bool short_q4k = m->gate->type == JQ_TYPE_Q4_K && c.hidden <= 2048 && c.inter <= 2048;
        // (Q4_K unpacks for less: a 256-token call of DeepSeek-V3-sized Q4_K experts, 3.8 ms, is 0.34 an expert)
        // (long rows: a = 0.07 + 0.17 bytes-per-weight; DeepSeek-V3 sizes, 8 tokens: 4.9 us a pair of IQ2_XXS, 6.7 of MXFP4)
        const double a = (short_q4k ? 0.10 : 0.07) + 0.17 * bpw, g = short_q4k ? 0.28 : m->gate->type == JQ_TYPE_Q4_K ? 0.36 : 0.30;
        const double hit = (double)c.n_expert * (1.0 - std::pow(1.0 - 1.0 / (double)c.n_expert, (double)P));
        const double by_pairs = (double)P * a, by_gemm = hit * g;
        double by_expert = INFINITY;
        if (has_expert_dot8 && !expert_env)
            by_expert = 0.10 * (hit + extra) + 0.032 * (double)(P + extra * (int)T) + 90e6 / (3.0 * c.hidden * (double)c.inter);
        decode_sized = by_pairs <= std::min(by_gemm, by_expert) && P <= 16384;
        if (!expert_env) expert_dot8 = by_expert < by_gemm;
    }
    bool planes_ready = false;
    jq::MoeGateIn gate_later{};
    if (decode_sized) {  // one group per pair, written by the gating kernel itself
        // long rows: the gate and up kernel reads x as fixed-point planes, which the router kernel can leave behind
        jq::ActsI8 planes{nullptr, nullptr, nullptr, nullptr};
        static const char *no_router_planes = getenv("JQ_MOE_NO_ROUTER_PLANES");
        if (!no_router_planes && m->gate->type == m->up->type && m->gate->row_bytes == m->up->row_bytes &&
            ((uintptr_t)x & 15) == 0 && !moe_gate_up_mfma_takes(m, x) &&
            moe_dot8_takes_planes(m->gate->type, m->gate->row_bytes, (((uintptr_t)m->gate->dev | (uintptr_t)m->up->dev) & 15) ? 4 : 16,
                                  (int)c.hidden, (int)c.inter, m->qi8))
            planes = m->qi8;
        // the matrix-core gate and up kernel can run the gating itself
        static const char *no_late_gate = getenv("JQ_MOE_NO_GATING_IN_GATE_UP");
        const bool late = !no_late_gate && m->gate->type == m->up->type && moe_gate_up_mfma_takes(m, x);
        // one token of a decoder layer: the norm in front of the experts runs inside the router launch
        static const char *no_pre = getenv("JQ_MOE_NO_NORM_IN_ROUTER");
        if (pre) {
            pre->fused = !no_pre && T == 1 && !planes.xl && c.hidden % 4 == 0 && x == pre->a.hn_out &&
                         (((uintptr_t)pre->a.x | (uintptr_t)pre->a.res | (uintptr_t)pre->a.w | (uintptr_t)pre->a.x_out |
                           (uintptr_t)pre->a.hn_out | (uintptr_t)m->router_w) & 15) == 0;
            if (!pre->fused)
                hipLaunchKernelGGL(jq::rmsnorm_rows, dim3((unsigned)T), dim3(1024), 0, s, (float *)pre->a.x, pre->a.res, pre->a.w,
                                   pre->a.eps, pre->a.hn_out, (int)c.hidden);
        }
        if (moe_route_dev(m, T, x, s, jq::MoePairGroups{m->gexp, m->offsets, m->xrow, m->yrow, extra}, planes, &planes_ready,
                          late ? &gate_later : nullptr, pre && pre->fused ? &pre->a : nullptr))
            return 1;
        groups = P + extra * (int)T;
        max_group = 1;
    } else {
        if (pre) {
            pre->fused = false;
            hipLaunchKernelGGL(jq::rmsnorm_rows, dim3((unsigned)T), dim3(1024), 0, s, (float *)pre->a.x, pre->a.res, pre->a.w,
                               pre->a.eps, pre->a.hn_out, (int)c.hidden);
        }
        // few pairs an expert of Q4_K with short rows: gate and up will run on the kernel that takes four rows an MFMA,
        // which reads x as fixed-point planes; the router launch leaves them behind
        jq::ActsI8 planes{nullptr, nullptr, nullptr, nullptr};
        {
            const jq_weight *ws[4] = {m->gate, m->up, m->fold_shared ? m->sgate : nullptr, m->fold_shared ? m->sup : nullptr};
            uintptr_t bits = 0;
            for (const jq_weight *w : ws) bits |= w ? ((uintptr_t)w->dev | (uintptr_t)w->row_bytes) : 0;
            static const char *no_router_planes = getenv("JQ_MOE_NO_ROUTER_PLANES");
            if (!no_router_planes && !expert_dot8 && m->gate->type == JQ_TYPE_Q4_K && m->up->type == JQ_TYPE_Q4_K &&
                m->gate->row_bytes == m->up->row_bytes && (size_t)P <= 6 * (size_t)c.n_expert &&
                moe_q4k_quads_takes(m->qi8, m->gate->row_bytes, (bits & 15) ? 4 : 16, x, (int)c.hidden))
                planes = m->qi8;
        }
        if (moe_route_dev(m, T, x, s, jq::MoePairGroups{nullptr, nullptr, nullptr, nullptr, 0}, planes, &planes_ready)) return 1;
        groups = (int)c.n_expert + extra;
        max_group = (int)T;
        const int in_lds = (size_t)P <= 12288;
        const size_t chunks = ((size_t)P + 63) / 64, rank_ints = chunks * c.n_expert + c.n_expert + 1;
        static const char *no_ranked = getenv("JQ_MOE_NO_RANKED_GROUPING");
        // (its rank table: chunks x experts ints of LDS, up to 144 KB)
        if (!no_ranked && chunks <= (size_t)jq::GROUP_RANK_CHUNKS && rank_ints <= 36864) {
            static std::once_flag big_lds;
            static hipError_t attr_rc = hipSuccess;
            std::call_once(big_lds, [&] {
                attr_rc = hipFuncSetAttribute((const void *)jq::moe_group_pairs_ranked, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              36864 * (int)sizeof(int));
            });
            HIP_TRY(attr_rc);
            hipLaunchKernelGGL(jq::moe_group_pairs_ranked, dim3(1), dim3(jq::GROUP_PAIRS_THREADS), rank_ints * sizeof(int), s,
                               m->ids, (int)T, (int)c.n_expert_used, (int)c.n_expert, m->gexp, m->offsets, m->xrow, m->yrow,
                               extra);
        }
        else
            hipLaunchKernelGGL(jq::moe_group_pairs, dim3(1), dim3(jq::GROUP_PAIRS_THREADS), (c.n_expert + 1 + (in_lds ? P : 0)) * sizeof(int), s,
                               m->ids, (int)T, (int)c.n_expert_used, (int)c.n_expert, m->gexp, m->offsets, m->xrow, m->yrow,
                               extra, in_lds);
    }
    HIP_TRY(hipGetLastError());
    // silu(gate x) * (up x) of every pair into G, then down over it
    // What every expert's first byte is a multiple of (a view may start at any whole block, and blocks of 17,
    // 34, 66, 210 bytes put that anywhere): 16-byte and 4-byte loads into LDS want it, the kernels that read
    // through registers do not.
    auto align_of = [](std::initializer_list<const jq_weight *> ws) {
        uintptr_t bits = 0;
        for (const jq_weight *w : ws)
            if (w) bits |= (uintptr_t)w->dev;
        return (bits & 15) == 0 ? 16 : (bits & 3) == 0 ? 4 : 1;
    };
    const int a16 = align_of({m->gate, m->up, m->fold_shared ? m->sgate : nullptr, m->fold_shared ? m->sup : nullptr});
    int rc = -1;
    const bool same_gu = m->gate->type == m->up->type && m->gate->row_bytes == m->up->row_bytes;
    // few tokens an expert (at most six on average): the int8 kernel that takes four rows an MFMA; more: the
    // f16 ring kernel, which reads a group's weights once for up to 16 rows
    const bool few = (size_t)P <= 6 * (size_t)c.n_expert;
    // many tokens an expert (16 on average or more): the grouped int8 GEMM, which unpacks a weight tile once for
    // 128 rows (Qwen3-30B-A3B sizes, evenly routed tokens: 352 us a call of 256 tokens against the ring kernel's 324,
    // 504 against 526 at 512, 1.19 ms against 2.03 at 2048).  The ring kernel walks an expert's rows once per 16 of its
    // pairs, so its time follows the fullest expert, which the host does not know: 512 copies of one token (8 experts
    // with 512 pairs each) take it 2.45 ms a layer and the GEMM 0.7, hence the GEMM from where the two are level.
    static const char *gemm_from_env = getenv("JQ_MOE_GEMM_FROM_PAIRS_PER_EXPERT");
    const size_t gemm_from = gemm_from_env ? (size_t)atoll(gemm_from_env) : 16;
    const bool prefer_gemm = m->gacts && max_group > 1 && (size_t)P >= gemm_from * (size_t)c.n_expert &&
                             c.hidden % 256 == 0 && c.inter % 256 == 0 && a16 >= 16 &&
                             align_of({m->down, m->fold_shared ? m->sdown : nullptr}) >= 16;
    // few pairs an expert, by the cost estimate above: the expert's rows decoded once, its pairs streamed past
    const bool multi = max_group > 1 && expert_dot8;
    if (same_gu && multi)
        rc = dispatch_moe_expert_dot8<true>(m->gate->type, m->pgate, m->pup, m->gate->row_bytes, a16, x, T, m->qi8, m->gexp,
                                            m->offsets, m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, s, clamp);
    if (rc > 0) return 1;
    if (rc < 0 && same_gu && max_group > 1 && m->gate->type == JQ_TYPE_Q4_K && few)
        rc = dispatch_moe_q4k_quads<true>(m->pgate, m->pup, m->gate->row_bytes, a16, x, T, m->qi8, m->gexp, m->offsets,
                                          m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, s, clamp,
                                          max_group > 1 && planes_ready);
    if (rc > 0) return 1;
    if (rc < 0 && same_gu && max_group > 1 && m->gate->type == JQ_TYPE_Q4_K && !prefer_gemm)
        rc = dispatch_moe_q4k_ring<true>(m->pgate, m->pup, m->gate->row_bytes, a16, x, T, m->qacts, m->gexp, m->offsets,
                                         m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, s, clamp);
    if (rc > 0) return 1;
    // bucketed, any format with a side of the int8 GEMM: gate -> G and up -> U from one preparation of x, then
    // the activation in place
    bool planned = false;
    if (rc < 0 && same_gu && max_group > 1 && m->gacts) {
        moe_gemm_plan(m, groups, (size_t)P + (size_t)extra * T, s);
        planned = true;
        rc = dispatch_moe_gemm_i8(m, m->gate->type, m->pgate, m->gate->row_bytes, a16, x, m->xrow, false, m->G, (int)c.hidden,
                                  (int)c.inter, s);
        if (rc == 0) {
            if (dispatch_moe_gemm_i8(m, m->up->type, m->pup, m->up->row_bytes, a16, x, m->xrow, true, m->U, (int)c.hidden,
                                     (int)c.inter, s) != 0)
                return fail("moe: the grouped GEMM took the gate projection and not the up projection");
            const size_t routed = (size_t)P * c.inter, folded = (size_t)extra * T * c.inter;
            hipLaunchKernelGGL(jq::swiglu_in_place, dim3((unsigned)std::min<size_t>((routed + 255) / 256, 4096)), dim3(256), 0,
                               s, m->G, m->U, routed, c.swiglu_clamp);
            if (folded)
                hipLaunchKernelGGL(jq::swiglu_in_place, dim3((unsigned)std::min<size_t>((folded + 255) / 256, 4096)), dim3(256),
                                   0, s, m->G + routed, m->U + routed, folded, c.swiglu_clamp_shared);
        }
    }
    if (rc > 0) return 1;
    // decode-sized Q4_K: the matrix-core kernels; a call of few row tiles clears y here and lets two workgroups a
    // tile add into it in the down projection
    bool y_cleared = false;
    if (rc < 0 && same_gu && max_group <= 1) {
        const bool will_split = (m->fold_shared || !m->sgate) && c.hidden <= 2048 && c.hidden % 16 == 0 &&
                                (m->down->type == JQ_TYPE_Q4_K || (m->down->type == JQ_TYPE_Q6_K && c.inter == 768)) &&
                                moe_down_mfma_splits(m, (int)T, extra);
        rc = dispatch_moe_gate_up_mfma(m, x, groups, s, clamp, will_split ? y : nullptr, will_split ? (int)(T * c.hidden) : 0,
                                       gate_later.logits ? &gate_later : nullptr);
        if (rc < 0 && gate_later.logits) return fail("moe: the gating was left to a kernel that declined the call");
        y_cleared = rc == 0 && will_split;
    }
    if (rc > 0) return 1;
    if (rc < 0 && same_gu && max_group <= 1)
        rc = dispatch_moe_dot8<true>(m->gate->type, m->pgate, m->pup, m->gate->row_bytes, a16, x, T, m->qi8, m->gexp,
                                     m->offsets, m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, s, clamp,
                                     planes_ready);
    if (rc > 0) return 1;
    if (rc < 0 && same_gu)
        rc = dispatch_moe_staged<true>(m->gate->type, m->pgate, m->pup, m->gate->row_bytes, a16, x, m->gexp, m->offsets,
                                       m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, max_group, s, clamp);
    if (rc > 0) return 1;
    const bool fused_act = rc == 0;
    if (!fused_act) {
        if (dispatch_moe_rows<false>(m->gate->type, m->pgate, m->gate->row_bytes, x, nullptr, m->gexp, m->offsets,
                                     m->xrow, m->yrow, m->G, (int)c.hidden, (int)c.inter, groups, max_group, s))
            return 1;
        if (dispatch_moe_rows<false>(m->up->type, m->pup, m->up->row_bytes, x, nullptr, m->gexp, m->offsets, m->xrow,
                                     m->yrow, m->U, (int)c.hidden, (int)c.inter, groups, max_group, s))
            return 1;
    }
    const int d16 = align_of({m->down, m->fold_shared ? m->sdown : nullptr});
    rc = -1;
    if (fused_act && multi)
        rc = dispatch_moe_expert_dot8<false>(m->down->type, m->pdown, nullptr, m->down->row_bytes, d16, m->G,
                                             (size_t)P + extra * T, m->qi8, m->gexp, m->offsets, m->yrow, m->yrow, m->out,
                                             (int)c.inter, (int)c.hidden, groups, s);
    if (rc > 0) return 1;
    // (where gate and up ran on the grouped GEMM, their rows being too long for the Q4_K kernels for short rows, so does
    // the down projection: those kernels walk an expert's 7168 rows at DeepSeek-V3 sizes, 7.7 ms a call of 256 tokens)
    if (rc < 0 && fused_act && max_group > 1 && m->down->type == JQ_TYPE_Q4_K && few && !planned)
        rc = dispatch_moe_q4k_quads<false>(m->pdown, nullptr, m->down->row_bytes, d16, m->G, (size_t)P + extra * T,
                                           m->qi8, m->gexp, m->offsets, m->yrow, m->yrow, m->out, (int)c.inter,
                                           (int)c.hidden, groups, s);
    if (rc > 0) return 1;
    if (rc < 0 && fused_act && max_group > 1 && m->down->type == JQ_TYPE_Q4_K && !prefer_gemm && !planned)
        rc = dispatch_moe_q4k_ring<false>(m->pdown, nullptr, m->down->row_bytes, d16, m->G, (size_t)P + extra * T,
                                          m->qacts, m->gexp, m->offsets, m->yrow, m->yrow, m->out, (int)c.inter,
                                          (int)c.hidden, groups, s);
    if (rc > 0) return 1;
    if (rc < 0 && fused_act && max_group > 1 && m->gacts) {
        if (!planned) moe_gemm_plan(m, groups, (size_t)P + (size_t)extra * T, s);
        rc = dispatch_moe_gemm_i8(m, m->down->type, m->pdown, m->down->row_bytes, d16, m->G, m->yrow, false, m->out,
                                  (int)c.inter, (int)c.hidden, s);
    }
    if (rc > 0) return 1;
    // decode-sized, and no shared expert outside the pair list: down projection and combine in one launch
    if (rc < 0 && fused_act && max_group <= 1 && (m->fold_shared || !m->sgate)) {
        rc = dispatch_moe_down_mfma(m, m->G, y, (int)T, extra, y_cleared, s);
        if (rc == 0) return 0;
        if (rc > 0) return 1;
        rc = dispatch_moe_down_combine(m->down->type, m->pdown, m->down->row_bytes, d16, m->G, (size_t)P + extra * T, m->qi8,
                                       m->gexp, m->wts, y, (int)c.inter, (int)c.hidden, (int)T, (int)c.n_expert_used, extra, s);
        if (rc == 0) return 0;
    }
    if (rc > 0) return 1;
    if (rc < 0 && fused_act && max_group <= 1)
        rc = dispatch_moe_dot8<false>(m->down->type, m->pdown, nullptr, m->down->row_bytes, d16, m->G, (size_t)P + extra * T,
                                      m->qi8, m->gexp, m->offsets, m->yrow, m->yrow, m->out, (int)c.inter, (int)c.hidden,
                                      groups, s);
    if (rc > 0) return 1;
    if (rc < 0 && fused_act)
        rc = dispatch_moe_staged<false>(m->down->type, m->pdown, nullptr, m->down->row_bytes, d16, m->G, m->gexp,
                                        m->offsets, m->yrow, m->yrow, m->out, (int)c.inter, (int)c.hidden, groups,
                                        max_group, s);
    if (rc > 0) return 1;
    if (rc < 0) {
        if (fused_act) {  // G already holds the activation: plain rows over it
            if (dispatch_moe_rows<false>(m->down->type, m->pdown, m->down->row_bytes, m->G, nullptr, m->gexp, m->offsets,
                                         m->yrow, m->yrow, m->out, (int)c.inter, (int)c.hidden, groups, max_group, s))
                return 1;
        } else if (dispatch_moe_rows<true>(m->down->type, m->pdown, m->down->row_bytes, m->G, m->U, m->gexp, m->offsets,
                                           m->yrow, m->yrow, m->out, (int)c.inter, (int)c.hidden, groups, max_group, s,
                                           clamp)) {
            return 1;
        }
    }
    const float *shared_out = nullptr;
    if (m->fold_shared) {
        shared_out = m->out + (size_t)P * c.hidden;  // the rows the shared expert's pairs wrote
    } else if (m->sgate) {  // shared expert over every token (reference: src/quantized_deepseek2.rs:555-557)
        size_t si = m->sgate->n;
        if (dispatch_matmul(m->sgate->type, m->sgate->dev, m->sgate->row_bytes, x, m->sG, T, c.hidden, si, s)) return 1;
        if (dispatch_matmul(m->sup->type, m->sup->dev, m->sup->row_bytes, x, m->sU, T, c.hidden, si, s)) return 1;
        size_t total = T * si;
        hipLaunchKernelGGL(jq::swiglu_rows, dim3((unsigned)std::min<size_t>((total + 255) / 256, 4096)), dim3(256), 0, s,
                           m->sG, m->sU, m->sH, total, c.swiglu_clamp_shared);
        if (dispatch_matmul(m->sdown->type, m->sdown->dev, m->sdown->row_bytes, m->sH, m->sOut, T, si, c.hidden, s))
            return 1;
        shared_out = m->sOut;
    }
    size_t total = T * c.hidden;
    hipLaunchKernelGGL(jq::moe_combine, dim3((unsigned)std::min<size_t>((total + 255) / 256, 4096)), dim3(256), 0, s,
                       m->out, m->wts, (int)T, (int)c.n_expert_used, (int)c.hidden, shared_out, y);
    HIP_TRY(hipGetLastError());
    return 0;
}

// Device table of expert base pointers; `extra` (the shared expert's weight, or null) becomes entry
// n_expert.
int moe_ptr_table(const jq_weight *w, size_t n_expert, size_t rows_per_expert, const jq_weight *extra,
                  const uint8_t ***out) {
    std::vector<const uint8_t *> host(n_expert + 1);
    for (size_t e = 0; e < n_expert; e++) host[e] = w->dev + e * rows_per_expert * w->row_bytes;
    host[n_expert] = extra ? extra->dev : w->dev;
    HIP_TRY(hipMalloc((void **)out, host.size() * sizeof(uint8_t *)));
    HIP_TRY(hipMemcpy((void *)*out, host.data(), host.size() * sizeof(uint8_t *), hipMemcpyHostToDevice));
    return 0;
}

}  // namespace

extern "C" {

int jq_moe_create(const jq_moe_config *cfg, const float *router_w, const float *router_bias,
                  const jq_weight *gate_exps, const jq_weight *up_exps, const jq_weight *down_exps,
                  const jq_weight *shared_gate, const jq_weight *shared_up, const jq_weight *shared_down,
                  jq_moe **out) {
    if (!out) return fail("jq_moe_create: out is null");
    *out = nullptr;
    if (!cfg || !router_w || !gate_exps || !up_exps || !down_exps) return fail("jq_moe_create: null argument");
    const jq_moe_config &c = *cfg;
    if (c.n_expert == 0 || c.n_expert_used == 0 || c.n_expert_used > c.n_expert)
        return fail("moe: %u experts used of %u", c.n_expert_used, c.n_expert);
    if (c.hidden % 4 != 0) return fail("moe: hidden size %u is not a multiple of 4", c.hidden);
    if (c.n_group > 1 && (c.n_expert % c.n_group != 0 || c.topk_group == 0 || c.topk_group > c.n_group))
        return fail("moe: %u experts in %u groups, %u groups kept", c.n_expert, c.n_group, c.topk_group);
    // reference: src/quantized_qwen3_moe.rs:567-571 (expert tensor shaped [n_expert, out, in])
    if (gate_exps->n != (size_t)c.n_expert * c.inter || gate_exps->k != c.hidden || up_exps->n != gate_exps->n ||
        up_exps->k != c.hidden || down_exps->n != (size_t)c.n_expert * c.hidden || down_exps->k != c.inter)
        return fail("moe: expected expert tensors shaped [%u*%u, %u], [%u*%u, %u], [%u*%u, %u]", c.n_expert, c.inter,
                    c.hidden, c.n_expert, c.inter, c.hidden, c.n_expert, c.hidden, c.inter);
    bool any_shared = shared_gate || shared_up || shared_down;
    if (any_shared) {
        if (!(shared_gate && shared_up && shared_down)) return fail("moe: shared expert needs gate, up and down");
        if (shared_gate->k != c.hidden || shared_up->k != c.hidden || shared_up->n != shared_gate->n ||
            shared_down->k != shared_gate->n || shared_down->n != c.hidden)
            return fail("moe: shared expert shapes do not chain");
    }
    if (ensure_init()) return 1;
    jq_moe *m = new jq_moe;
    m->cfg = c;
    m->gate = gate_exps;
    m->up = up_exps;
    m->down = down_exps;
    m->sgate = shared_gate;
    m->sup = shared_up;
    m->sdown = shared_down;
    auto cleanup = [&] {
        jq_moe_free(m);
        return 1;
    };
    size_t rbytes = (size_t)c.n_expert * c.hidden * sizeof(float);
    if (hipMalloc((void **)&m->router_w, rbytes) != hipSuccess ||
        hipMemcpy(m->router_w, router_w, rbytes, hipMemcpyHostToDevice) != hipSuccess) {
        fail("moe: router upload failed");
        return cleanup();
    }
    if (router_bias) {
        if (hipMalloc((void **)&m->router_bias, c.n_expert * sizeof(float)) != hipSuccess ||
            hipMemcpy(m->router_bias, router_bias, c.n_expert * sizeof(float), hipMemcpyHostToDevice) != hipSuccess) {
            fail("moe: router bias upload failed");
            return cleanup();
        }
    }
    // A shared expert of the routed experts' own type and shape rides along in the grouped kernels.
    m->fold_shared = any_shared && shared_gate->type == gate_exps->type && shared_up->type == up_exps->type &&
                     shared_down->type == down_exps->type && shared_gate->n == c.inter;
    if (moe_ptr_table(gate_exps, c.n_expert, c.inter, m->fold_shared ? shared_gate : nullptr, &m->pgate) ||
        moe_ptr_table(up_exps, c.n_expert, c.inter, m->fold_shared ? shared_up : nullptr, &m->pup) ||
        moe_ptr_table(down_exps, c.n_expert, c.hidden, m->fold_shared ? shared_down : nullptr, &m->pdown))
        return cleanup();
    *out = m;
    return 0;
}

void jq_moe_free(jq_moe *m) {
    if (!m) return;
    moe_free_scratch(m);
    for (void *p : {(void *)m->router_w, (void *)m->router_bias, (void *)m->pgate, (void *)m->pup, (void *)m->pdown})
        if (p) (void)hipFree(p);
    delete m;
}

int jq_moe_route(jq_moe *m, size_t n_tokens, const float *x, uint32_t *ids, float *weights, int ptrs_are_device,
                 void *stream) {
    if (!m) return fail("jq_moe_route: layer is null");
    if (n_tokens == 0) return 0;
    if (!x || !ids || !weights) return fail("jq_moe_route: null pointer");
    hipStream_t s = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(m->mu);
    if (moe_reserve(m, n_tokens)) return 1;
    size_t P = n_tokens * m->cfg.n_expert_used;
    DevBuf xd;
    const float *xdev = x;
    if (!ptrs_are_device) {
        HIP_TRY(xd.alloc(n_tokens * m->cfg.hidden * sizeof(float)));
        HIP_TRY(hipMemcpyAsync(xd.p, x, n_tokens * m->cfg.hidden * sizeof(float), hipMemcpyHostToDevice, s));
        xdev = (const float *)xd.p;
    }
    if (moe_route_dev(m, n_tokens, xdev, s, jq::MoePairGroups{nullptr, nullptr, nullptr, nullptr, 0})) return 1;
    hipMemcpyKind kind = ptrs_are_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost;
    HIP_TRY(hipMemcpyAsync(ids, m->ids, P * sizeof(uint32_t), kind, s));
    HIP_TRY(hipMemcpyAsync(weights, m->wts, P * sizeof(float), kind, s));
    if (!ptrs_are_device) HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int jq_moe_forward(jq_moe *m, size_t n_tokens, const float *x, float *y, int ptrs_are_device, void *stream) {
    if (!m) return fail("jq_moe_forward: layer is null");
    if (n_tokens == 0) return 0;
    if (!x || !y) return fail("jq_moe_forward: null pointer");
    hipStream_t s = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(m->mu);
    if (moe_reserve(m, n_tokens)) return 1;
    if (ptrs_are_device) return moe_forward_dev(m, n_tokens, x, y, s);
    size_t bytes = n_tokens * m->cfg.hidden * sizeof(float);
    DevBuf xd, yd;
    HIP_TRY(xd.alloc(bytes));
    HIP_TRY(yd.alloc(bytes));
    HIP_TRY(hipMemcpyAsync(xd.p, x, bytes, hipMemcpyHostToDevice, s));
    if (moe_forward_dev(m, n_tokens, (const float *)xd.p, (float *)yd.p, s)) return 1;
    HIP_TRY(hipMemcpyAsync(y, yd.p, bytes, hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

}  // extern "C"

// ---- multi-head latent attention -----------------------------------------------------

struct jq_mla {
    jq_mla_config cfg;
    const jq_weight *q, *q_b, *kv_a, *kv_b, *o;
    float *q_a_norm = nullptr, *kv_a_norm = nullptr;
    float *wkv = nullptr;   // the KV up-projection as dense f32 [n_head * (nope + vh), lkv]
    uint8_t *qa_kva = nullptr;  // q_a's rows followed by kv_a's in one allocation (same format and width): one product a single-token step
    float *qa_kva_out = nullptr;  // its result, q_lora_rank + lkv + rope floats
    float2 *cs = nullptr;   // [n_ctx][rope / 2] (cos, sin), scaled by the YaRN mscale
    float *lat = nullptr, *kpe = nullptr;  // the cache: [n_ctx][lkv] normed latents, [n_ctx][rope] rotated keys
    float scale = 0.0f;
    size_t n_past = 0;
    // scratch, grown to the largest token count seen
    size_t cap_tokens = 0;
    float *t1 = nullptr, *t1n = nullptr, *qv = nullptr, *comp = nullptr, *qabs = nullptr, *part = nullptr, *ctx = nullptr;
    std::vector<void *> retired;  // outgrown scratch, kept until the object goes
    std::mutex mu;
};

namespace {

constexpr size_t MLA_PART_SLOTS = 64;  // partial results kept per head: tokens of a call x context splits

void mla_free_scratch(jq_mla *m) {
    for (void *p : {(void *)m->t1, (void *)m->t1n, (void *)m->qv, (void *)m->comp, (void *)m->qabs, (void *)m->part, (void *)m->ctx})
        if (p) (void)hipFree(p);
    for (void *p : m->retired) (void)hipFree(p);
    m->retired.clear();
    m->t1 = m->t1n = m->qv = m->comp = m->qabs = m->part = m->ctx = nullptr;
    m->cap_tokens = 0;
}

// Scratch for calls of up to T tokens.  Buffers that are outgrown are retired, not freed: a HIP graph captured
// over an earlier, smaller call still names them, and they go with the object (jq_mla_free).
int mla_reserve(jq_mla *m, size_t T) {
    if (T <= m->cap_tokens) return 0;
    for (void *p : {(void *)m->t1, (void *)m->t1n, (void *)m->qv, (void *)m->comp, (void *)m->qabs, (void *)m->part, (void *)m->ctx})
        if (p) m->retired.push_back(p);
    m->t1 = m->t1n = m->qv = m->comp = m->qabs = m->part = m->ctx = nullptr;
    m->cap_tokens = 0;
    const jq_mla_config &c = m->cfg;
    const size_t qd = c.qk_nope_head_dim + c.qk_rope_head_dim;
    if (c.q_lora_rank) {
        HIP_TRY(hipMalloc((void **)&m->t1, T * c.q_lora_rank * sizeof(float)));
        HIP_TRY(hipMalloc((void **)&m->t1n, T * c.q_lora_rank * sizeof(float)));
    }
    HIP_TRY(hipMalloc((void **)&m->qv, T * c.n_head * qd * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->comp, T * (c.kv_lora_rank + c.qk_rope_head_dim) * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->qabs, T * c.n_head * c.kv_lora_rank * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->part, std::max(T, MLA_PART_SLOTS) * c.n_head * (c.kv_lora_rank + 2) * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->ctx, T * c.n_head * c.v_head_dim * sizeof(float)));
    m->cap_tokens = T;
    return 0;
}

// YaRN helpers in f32, as the reference computes them (src/quantized_deepseek2.rs:230-236, :314-339).
float yarn_get_mscale(float scale, float mscale) { return scale <= 1.0f ? 1.0f : 0.1f * mscale * logf(scale) + 1.0f; }
float yarn_find_correction_dim(float num_rot, size_t dim, float base, size_t max_pos) {
    return ((float)dim * logf((float)max_pos / (num_rot * 2.0f * 3.14159265358979323846f))) / (2.0f * logf(base));
}

// (cos, sin) of every position and rotary pair, scaled by mscale (src/quantized_deepseek2.rs:246-301).
std::vector<float2> mla_rope_table(const jq_mla_config &c) {
    const size_t dim = c.qk_rope_head_dim, half = dim / 2;
    std::vector<float> inv(half);
    float mscale = 1.0f;
    for (size_t i = 0; i < half; i++) inv[i] = 1.0f / powf(c.rope_theta, (float)(2 * i) / (float)dim);
    if (c.yarn_factor > 0.0f) {
        float lo = floorf(yarn_find_correction_dim(32.0f, dim, c.rope_theta, c.yarn_orig_context_length));
        float hi = ceilf(yarn_find_correction_dim(1.0f, dim, c.rope_theta, c.yarn_orig_context_length));
        lo = std::max(lo, 0.0f), hi = std::min(hi, (float)dim - 1.0f);
        if (fabsf(lo - hi) < 1.1920929e-7f) hi += 0.001f;
        for (size_t i = 0; i < half; i++) {
            const float extra = inv[i], inter = 1.0f / (c.yarn_factor * powf(c.rope_theta, (float)(2 * i) / (float)dim));
            const float ramp = std::min(std::max(((float)i - lo) / (hi - lo), 0.0f), 1.0f), mask = 1.0f - ramp;
            inv[i] = inter * (1.0f - mask) + extra * mask;
        }
        mscale = yarn_get_mscale(c.yarn_factor, c.yarn_mscale_all_dim);
    }
    std::vector<float2> cs((size_t)c.n_ctx * half);
    for (size_t t = 0; t < c.n_ctx; t++)
        for (size_t i = 0; i < half; i++) {
            const float f = (float)t * inv[i];
            cs[t * half + i] = float2{cosf(f) * mscale, sinf(f) * mscale};
        }
    return cs;
}

int mla_check_weight(const char *what, const jq_weight *w, size_t n, size_t k) {
    if (!w) return fail("jq_mla_create: %s is null", what);
    if (w->n != n || w->k != k) return fail("jq_mla_create: %s is [%zu, %zu], expected [%zu, %zu]", what, w->n, w->k, n, k);
    return 0;
}

template <int G>
int mla_launch_attention(const jq_mla *m, size_t S, size_t pos, unsigned n_split, hipStream_t s) {
    const jq_mla_config &c = m->cfg;
    const dim3 grid(c.n_head / G, n_split, (unsigned)S);
    const int lpl = (int)((c.kv_lora_rank + 63) / 64);
#define JQ_MLA_ATT(LPL)                                                                                              \
    hipLaunchKernelGGL((jq::mla_attention<G, LPL>), grid, dim3(256), 0, s, m->qabs, m->qv, m->lat, m->kpe, m->part, \
                       (int)c.n_head, (int)c.qk_nope_head_dim, (int)c.qk_rope_head_dim, (int)c.kv_lora_rank, (int)pos, \
                       (int)n_split, m->scale)
    if (lpl <= 1) JQ_MLA_ATT(1);
    else if (lpl <= 2) JQ_MLA_ATT(2);
    else if (lpl <= 4) JQ_MLA_ATT(4);
    else JQ_MLA_ATT(8);
#undef JQ_MLA_ATT
    HIP_TRY(hipGetLastError());
    return 0;
}

// x, out: device pointers; S tokens at positions pos .. pos + S - 1; scratch reserved for S.
int mla_forward_dev(jq_mla *m, size_t S, size_t pos, const float *x, float *out, hipStream_t s) {
    const jq_mla_config &c = m->cfg;
    const size_t nh = c.n_head, nope = c.qk_nope_head_dim, rope = c.qk_rope_head_dim, vh = c.v_head_dim,
                 lkv = c.kv_lora_rank, qd = nope + rope;
    const float *comp = m->comp;
    if (c.q_lora_rank) {
        float *t1 = m->t1;
        if (S == 1 && m->qa_kva) {  // one token: q_a and kv_a as one product over the rows laid end to end
            if (dispatch_matmul(m->q->type, m->qa_kva, m->q->row_bytes, x, m->qa_kva_out, 1, c.n_embd, m->q->n + m->kv_a->n, s)) return 1;
            t1 = m->qa_kva_out, comp = m->qa_kva_out + m->q->n;
        } else if (dispatch_matmul(m->q->type, m->q->dev, m->q->row_bytes, x, m->t1, S, c.n_embd, c.q_lora_rank, s)) {
            return 1;
        }
        hipLaunchKernelGGL(jq::rmsnorm_rows, dim3((unsigned)S), dim3(1024), 0, s, t1, (const float *)nullptr,
                           (const float *)m->q_a_norm, c.rms_eps, m->t1n, (int)c.q_lora_rank);
        HIP_TRY(hipGetLastError());
        if (dispatch_matmul(m->q_b->type, m->q_b->dev, m->q_b->row_bytes, m->t1n, m->qv, S, c.q_lora_rank, nh * qd, s)) return 1;
    } else if (dispatch_matmul(m->q->type, m->q->dev, m->q->row_bytes, x, m->qv, S, c.n_embd, nh * qd, s)) {
        return 1;
    }
    if (comp == m->comp && dispatch_matmul(m->kv_a->type, m->kv_a->dev, m->kv_a->row_bytes, x, m->comp, S, c.n_embd, lkv + rope, s))
        return 1;
    const bool vec4 = lkv % 4 == 0;
    const unsigned st = S == 1 ? 1 : 4;
    static const char *no_absorb_rope = getenv("JQ_MLA_NO_ABSORB_ROPE");
    if (S == 1 && !no_absorb_rope) {
        // one token: the rotation / latent kernel's work rides in the first wave of the absorption's workgroups
        if (vec4)
            hipLaunchKernelGGL(jq::mla_absorb_rope<4>, dim3((unsigned)nh + 1), dim3(512), 0, s, m->qv, (const float *)m->wkv, m->qabs,
                               (int)nh, (int)nope, (int)rope, (int)vh, (int)lkv, comp, (const float *)m->kv_a_norm,
                               (const float2 *)m->cs, m->lat, m->kpe, (int)pos, c.rms_eps);
        else
            hipLaunchKernelGGL(jq::mla_absorb_rope<1>, dim3((unsigned)nh + 1), dim3(512), 0, s, m->qv, (const float *)m->wkv, m->qabs,
                               (int)nh, (int)nope, (int)rope, (int)vh, (int)lkv, comp, (const float *)m->kv_a_norm,
                               (const float2 *)m->cs, m->lat, m->kpe, (int)pos, c.rms_eps);
        HIP_TRY(hipGetLastError());
    } else {
        hipLaunchKernelGGL(jq::mla_rope_latent, dim3((unsigned)nh + 1, (unsigned)S), dim3(64), 0, s, m->qv, comp,
                           (const float *)m->kv_a_norm, (const float2 *)m->cs, m->lat, m->kpe, (int)nh, (int)nope, (int)rope,
                           (int)lkv, (int)pos, c.rms_eps);
        HIP_TRY(hipGetLastError());
        // one token a workgroup in a decode step, four in a prefill; 16-byte loads when the latent width allows
        {
            const dim3 grid((unsigned)nh, (unsigned)((S + st - 1) / st));
#define JQ_MLA_ABSORB(ST, CW)                                                                                          \
        hipLaunchKernelGGL((jq::mla_absorb_q<ST, CW>), grid, dim3(512), 0, s, (const float *)m->qv, (const float *)m->wkv, \
                           m->qabs, (int)S, (int)nh, (int)nope, (int)rope, (int)vh, (int)lkv)
            if (vec4 && st == 1) JQ_MLA_ABSORB(1, 4);
            else if (vec4) JQ_MLA_ABSORB(4, 4);
            else if (st == 1) JQ_MLA_ABSORB(1, 1);
            else JQ_MLA_ABSORB(4, 1);
#undef JQ_MLA_ABSORB
            HIP_TRY(hipGetLastError());
        }
    }
    const size_t total = pos + S;
    size_t n_split;
    static const char *mla_env = getenv("JQ_MLA_ATTENTION");  // "valu": never the matrix-core kernel
    const bool mfma = lkv == jq::MLA_M_LKV && rope == jq::MLA_M_ROPE && nh % 32 == 0 && nope % 4 == 0 && !(mla_env && !strcmp(mla_env, "valu"));
    if (mfma) {
        // one workgroup a compute unit when the call has few tokens, tiles of 32 tokens
        const size_t wgs = S * (nh / 32);
        n_split = std::min<size_t>({(256 + wgs - 1) / wgs, (total + 31) / 32, (size_t)jq::MLA_SPLIT_MAX,
                                    std::max<size_t>(MLA_PART_SLOTS / S, 1)});
        static const char *split_env = getenv("JQ_MLA_SPLIT");
        if (split_env) n_split = std::min<size_t>(n_split, (size_t)atoi(split_env));
        n_split = std::max<size_t>(n_split, 1);
        hipLaunchKernelGGL(jq::mla_attention_mfma, dim3((unsigned)(nh / 32), (unsigned)n_split, (unsigned)S), dim3(512), 0, s,
                           (const float *)m->qabs, (const float *)m->qv, (const float *)m->lat, (const float *)m->kpe, m->part,
                           (int)nh, (int)nope, (int)pos, (int)n_split, m->scale);
        HIP_TRY(hipGetLastError());
    } else {
        // heads per workgroup, then enough context splits to fill the chip when the call has few tokens
        const int G = nh % 8 == 0 ? 8 : nh % 4 == 0 ? 4 : nh % 2 == 0 ? 2 : 1;
        const size_t wgs = S * (nh / G);
        n_split = std::min<size_t>({(1024 + wgs - 1) / wgs, (total + 31) / 32, (size_t)jq::MLA_SPLIT_MAX,
                                    std::max<size_t>(MLA_PART_SLOTS / S, 1)});
        n_split = std::max<size_t>(n_split, 1);
        int rc = G == 8 ? mla_launch_attention<8>(m, S, pos, (unsigned)n_split, s)
                 : G == 4 ? mla_launch_attention<4>(m, S, pos, (unsigned)n_split, s)
                 : G == 2 ? mla_launch_attention<2>(m, S, pos, (unsigned)n_split, s)
                          : mla_launch_attention<1>(m, S, pos, (unsigned)n_split, s);
        if (rc) return rc;
    }
    // the absorbed queries are spent: their buffer takes the merged latent sums
    hipLaunchKernelGGL(jq::mla_merge, dim3((unsigned)nh, (unsigned)S, (unsigned)((lkv + 127) / 128)), dim3(128), 0, s, (const float *)m->part, m->qabs, (int)nh,
                       (int)lkv, (int)n_split);
    HIP_TRY(hipGetLastError());
    {
        const dim3 grid((unsigned)nh, (unsigned)((vh + 15) / 16), (unsigned)((S + st - 1) / st));
#define JQ_MLA_VPROJ(ST, VEC)                                                                                          \
    hipLaunchKernelGGL((jq::mla_vproj<ST, VEC>), grid, dim3(256), 0, s, (const float *)m->qabs, (const float *)m->wkv, \
                       m->ctx, (int)S, (int)nh, (int)nope, (int)vh, (int)lkv)
        if (vec4 && st == 1) JQ_MLA_VPROJ(1, true);
        else if (vec4) JQ_MLA_VPROJ(4, true);
        else if (st == 1) JQ_MLA_VPROJ(1, false);
        else JQ_MLA_VPROJ(4, false);
#undef JQ_MLA_VPROJ
        HIP_TRY(hipGetLastError());
    }
    return dispatch_matmul(m->o->type, m->o->dev, m->o->row_bytes, m->ctx, out, S, nh * vh, c.n_embd, s);
}

}  // namespace

extern "C" {

int jq_mla_create(const jq_mla_config *cfg, const jq_weight *q_or_q_a, const float *q_a_norm, const jq_weight *q_b,
                  const jq_weight *kv_a_mqa, const float *kv_a_norm, const jq_weight *kv_b, const float *kv_b_dense,
                  const jq_weight *o_proj, jq_mla **out) {
    if (!cfg || !out) return fail("jq_mla_create: null argument");
    if (ensure_init()) return 1;
    const jq_mla_config &c = *cfg;
    const size_t nh = c.n_head, nope = c.qk_nope_head_dim, rope = c.qk_rope_head_dim, vh = c.v_head_dim,
                 lkv = c.kv_lora_rank, qd = nope + rope;
    if (!c.n_embd || !nh || !lkv || !rope || !vh || !c.n_ctx) return fail("jq_mla_create: a dimension is zero");
    if (rope % 2 != 0 || rope > 64) return fail("jq_mla_create: qk_rope_head_dim %zu must be even and at most 64", rope);
    if (lkv > (size_t)jq::MLA_MAX_LKV) return fail("jq_mla_create: kv_lora_rank %zu exceeds %d", lkv, jq::MLA_MAX_LKV);
    if (lkv % 4 != 0 && lkv > 128) return fail("jq_mla_create: kv_lora_rank %zu above 128 must be a multiple of 4", lkv);
    if (nope > (size_t)jq::MLA_MAX_NOPE) return fail("jq_mla_create: qk_nope_head_dim %zu exceeds %d", nope, jq::MLA_MAX_NOPE);
    if (c.q_lora_rank && (c.q_lora_rank % 4 != 0 || c.q_lora_rank > 8192))
        return fail("jq_mla_create: q_lora_rank %u must be a multiple of 4, at most 8192", c.q_lora_rank);
    if (c.yarn_factor > 0.0f && c.yarn_orig_context_length == 0) return fail("jq_mla_create: YaRN without an original context length");
    if (c.q_lora_rank) {
        if (mla_check_weight("attn_q_a", q_or_q_a, c.q_lora_rank, c.n_embd)) return 1;
        if (mla_check_weight("attn_q_b", q_b, nh * qd, c.q_lora_rank)) return 1;
        if (!q_a_norm) return fail("jq_mla_create: attn_q_a_norm is null");
    } else if (mla_check_weight("attn_q", q_or_q_a, nh * qd, c.n_embd)) {
        return 1;
    }
    if (mla_check_weight("attn_kv_a_mqa", kv_a_mqa, lkv + rope, c.n_embd)) return 1;
    if (!kv_a_norm) return fail("jq_mla_create: attn_kv_a_norm is null");
    if ((kv_b != nullptr) == (kv_b_dense != nullptr)) return fail("jq_mla_create: give attn_kv_b either quantized or dense");
    if (kv_b && mla_check_weight("attn_kv_b", kv_b, nh * (nope + vh), lkv)) return 1;
    if (mla_check_weight("attn_output", o_proj, c.n_embd, nh * vh)) return 1;

    std::unique_ptr<jq_mla, void (*)(jq_mla *)> m(new jq_mla, jq_mla_free);
    m->cfg = c;
    m->q = q_or_q_a, m->q_b = q_b, m->kv_a = kv_a_mqa, m->kv_b = kv_b, m->o = o_proj;
    double scale = 1.0 / sqrt((double)qd);  // f64 as in the reference (src/quantized_deepseek2.rs:186-192)
    if (c.yarn_factor > 0.0f) {
        const double ms = (double)yarn_get_mscale(c.yarn_factor, c.yarn_mscale_all_dim);
        scale *= ms * ms;
    }
    m->scale = (float)scale;
    const size_t wkv_elems = nh * (nope + vh) * lkv;
    HIP_TRY(hipMalloc((void **)&m->wkv, wkv_elems * sizeof(float)));
    if (kv_b) {
        if (dispatch_decode(kv_b, nullptr, m->wkv, kv_b->n, nullptr)) return 1;
    } else {
        HIP_TRY(hipMemcpy(m->wkv, kv_b_dense, wkv_elems * sizeof(float), hipMemcpyHostToDevice));
    }
    if (c.q_lora_rank) {
        HIP_TRY(hipMalloc((void **)&m->q_a_norm, c.q_lora_rank * sizeof(float)));
        HIP_TRY(hipMemcpy(m->q_a_norm, q_a_norm, c.q_lora_rank * sizeof(float), hipMemcpyHostToDevice));
    }
    HIP_TRY(hipMalloc((void **)&m->kv_a_norm, lkv * sizeof(float)));
    HIP_TRY(hipMemcpy(m->kv_a_norm, kv_a_norm, lkv * sizeof(float), hipMemcpyHostToDevice));
    if (c.q_lora_rank && m->q->type == m->kv_a->type && m->q->row_bytes == m->kv_a->row_bytes && !getenv("JQ_MLA_NO_FUSED_QA_KVA")) {
        const size_t qa_bytes = m->q->n * m->q->row_bytes, kva_bytes = m->kv_a->n * m->kv_a->row_bytes;
        HIP_TRY(hipMalloc((void **)&m->qa_kva, qa_bytes + kva_bytes));
        HIP_TRY(hipMemcpy(m->qa_kva, m->q->dev, qa_bytes, hipMemcpyDeviceToDevice));
        HIP_TRY(hipMemcpy(m->qa_kva + qa_bytes, m->kv_a->dev, kva_bytes, hipMemcpyDeviceToDevice));
        HIP_TRY(hipMalloc((void **)&m->qa_kva_out, (m->q->n + m->kv_a->n) * sizeof(float)));
    }
    const std::vector<float2> cs = mla_rope_table(c);
    HIP_TRY(hipMalloc((void **)&m->cs, cs.size() * sizeof(float2)));
    HIP_TRY(hipMemcpy(m->cs, cs.data(), cs.size() * sizeof(float2), hipMemcpyHostToDevice));
    HIP_TRY(hipMalloc((void **)&m->lat, (size_t)c.n_ctx * lkv * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->kpe, (size_t)c.n_ctx * rope * sizeof(float)));
    HIP_TRY(hipDeviceSynchronize());
    *out = m.release();
    return 0;
}

void jq_mla_free(jq_mla *m) {
    if (!m) return;
    mla_free_scratch(m);
    for (void *p : {(void *)m->q_a_norm, (void *)m->kv_a_norm, (void *)m->wkv, (void *)m->cs, (void *)m->lat, (void *)m->kpe,
                    (void *)m->qa_kva, (void *)m->qa_kva_out})
        if (p) (void)hipFree(p);
    delete m;
}

int jq_mla_forward(jq_mla *m, size_t n_tokens, size_t pos, const float *x, float *out, int ptrs_are_device, void *stream) {
    if (!m) return fail("jq_mla_forward: object is null");
    if (n_tokens == 0) return 0;
    if (!x || !out) return fail("jq_mla_forward: null pointer");
    std::lock_guard<std::mutex> lock(m->mu);
    if (pos != m->n_past) return fail("jq_mla_forward: pos %zu, but %zu tokens are cached", pos, m->n_past);
    if (pos + n_tokens > m->cfg.n_ctx) return fail("jq_mla_forward: %zu + %zu tokens exceed the context of %u", pos, n_tokens, m->cfg.n_ctx);
    if (n_tokens > 0x7FFF) return fail("jq_mla_forward: at most 32767 tokens a call");
    hipStream_t s = (hipStream_t)stream;
    if (mla_reserve(m, n_tokens)) return 1;
    const size_t bytes = n_tokens * m->cfg.n_embd * sizeof(float);
    if (ptrs_are_device) {
        if (mla_forward_dev(m, n_tokens, pos, x, out, s)) return 1;
    } else {
        DevBuf xd, yd;
        HIP_TRY(xd.alloc(bytes));
        HIP_TRY(yd.alloc(bytes));
        HIP_TRY(hipMemcpyAsync(xd.p, x, bytes, hipMemcpyHostToDevice, s));
        if (mla_forward_dev(m, n_tokens, pos, (const float *)xd.p, (float *)yd.p, s)) return 1;
        HIP_TRY(hipMemcpyAsync(out, yd.p, bytes, hipMemcpyDeviceToHost, s));
        HIP_TRY(hipStreamSynchronize(s));
    }
    m->n_past += n_tokens;
    return 0;
}

int jq_mla_reset(jq_mla *m) {
    if (!m) return fail("jq_mla_reset: object is null");
    std::lock_guard<std::mutex> lock(m->mu);
    m->n_past = 0;
    return 0;
}

size_t jq_mla_cached_tokens(const jq_mla *m) { return m ? m->n_past : 0; }

}  // extern "C"

// ---- dense Qwen3 decoder ------------------------------------------------------------

struct jq_model {
    jq_qwen3_config cfg;
    std::map<std::string, jq_weight *> q;   // quantized matrices by GGUF name
    std::map<std::string, float *> f;       // f32 vectors by GGUF name
    // Matrices that multiply the same activation, laid one after the other in one allocation
    // (blk.N.qkv, blk.N.gate_up): one launch for a single-token step; q holds views of their parts.
    std::map<std::string, jq_weight *> fused;
    std::set<std::string> paired;      // fused gate|up entries whose rows alternate gate_j, up_j (see model_fuse)
    std::vector<jq_weight *> retired;  // fused allocations whose parts were replaced; views may still point into them
    bool fused_ready = false;
    float *cat = nullptr;     // the fused result of a single-token step (q|k|v, gate|up)
    std::vector<float *> kc, vc;            // per layer [n_kv, n_ctx, d]
    uint32_t n_past = 0;
    size_t cap_tokens = 0;
    uint32_t *ids = nullptr, *pick = nullptr;
    float *pick_v = nullptr;  // the greedy pick's candidates, one per slice of the logits
    int *pick_i = nullptr;
    int *pos = nullptr;       // device copy of the position of the step being run
    float *part = nullptr;    // split-attention partials
    float2 *rope_cs = nullptr;  // (cos, sin) of the rotary angles of a step's tokens, [8][head_dim / 2]
    float *x2 = nullptr;      // second residual row of a single-token step (the fused norm + matmul launches alternate)
    float *x = nullptr, *hn = nullptr, *qb = nullptr, *kb = nullptr, *vb = nullptr, *att = nullptr, *proj = nullptr,
          *g = nullptr, *u = nullptr, *mid = nullptr, *logits = nullptr;
    // Mixture-of-experts feed-forward blocks (cfg.n_expert > 0): the routers as they arrived from the host,
    // one layer object each (built at the first step, rebuilt when a tensor of the layer is replaced), and
    // the index of the one that currently holds the scratch buffers all of them take turns with.
    std::map<std::string, std::vector<float>> router_host;
    std::vector<jq_moe *> moe;
    int moe_scratch_at = -1;
    std::mutex mu;
};

namespace {

// Hands the scratch buffers of one layer object to another of the same configuration.  Work on a stream
// runs in launch order and every kernel got its pointers when it was launched, so the layers of a model
// can take turns with one set.
void moe_swap_scratch(jq_moe *a, jq_moe *b) {
    std::swap(a->cap_tokens, b->cap_tokens);
    std::swap(a->logits, b->logits), std::swap(a->wts, b->wts), std::swap(a->G, b->G), std::swap(a->U, b->U);
    std::swap(a->out, b->out), std::swap(a->sG, b->sG), std::swap(a->sU, b->sU), std::swap(a->sH, b->sH);
    std::swap(a->sOut, b->sOut), std::swap(a->ids, b->ids), std::swap(a->gexp, b->gexp);
    std::swap(a->offsets, b->offsets), std::swap(a->xrow, b->xrow), std::swap(a->yrow, b->yrow);
    std::swap(a->qacts, b->qacts), std::swap(a->gacts, b->gacts), std::swap(a->gtab, b->gtab);
    std::swap(a->gtab_rows, b->gtab_rows), std::swap(a->gtile_rgs, b->gtile_rgs), std::swap(a->qi8, b->qi8);
}

void model_free_scratch(jq_model *m) {
    for (void *p : {(void *)m->ids, (void *)m->x, (void *)m->x2, (void *)m->hn, (void *)m->qb, (void *)m->kb, (void *)m->vb,
                    (void *)m->att, (void *)m->proj, (void *)m->g, (void *)m->mid})  // u is the second half of g
        if (p) (void)hipFree(p);
    m->ids = nullptr;
    m->x2 = nullptr;
    m->x = m->hn = m->qb = m->kb = m->vb = m->att = m->proj = m->g = m->u = m->mid = nullptr;
    m->cap_tokens = 0;
}

int model_reserve(jq_model *m, size_t T) {
    if (T <= m->cap_tokens) return 0;
    model_free_scratch(m);
    const jq_qwen3_config &c = m->cfg;
    size_t qd = (size_t)c.n_head * c.head_dim, kd = (size_t)c.n_kv_head * c.head_dim;
    HIP_TRY(hipMalloc((void **)&m->ids, T * sizeof(uint32_t)));
    HIP_TRY(hipMalloc((void **)&m->x, T * c.hidden * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->x2, c.hidden * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->hn, T * c.hidden * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->qb, T * (qd + 2 * kd) * sizeof(float)));  // q, or the rows of one q|k|v product
    HIP_TRY(hipMalloc((void **)&m->kb, T * kd * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->vb, T * kd * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->att, T * qd * sizeof(float)));
    HIP_TRY(hipMalloc((void **)&m->proj, T * c.hidden * sizeof(float)));
    // gate and up results in one allocation: a many-token step over a paired gate|up matrix writes its
    // T x 2 ffn result (gate_j, up_j alternating) across both
    HIP_TRY(hipMalloc((void **)&m->g, 2 * T * c.ffn * sizeof(float)));
    m->u = m->g + T * c.ffn;
    HIP_TRY(hipMalloc((void **)&m->mid, T * c.ffn * sizeof(float)));
    m->cap_tokens = T;
    return 0;
}

// Expected [n, k] of a tensor name; k == 0 marks an f32 vector of length n.
bool qwen3_shape(const jq_qwen3_config &c, const std::string &name, size_t *n, size_t *k) {
    size_t qd = (size_t)c.n_head * c.head_dim, kd = (size_t)c.n_kv_head * c.head_dim;
    auto ends = [&](const char *suf) {
        size_t l = strlen(suf);
        return name.size() >= l && name.compare(name.size() - l, l, suf) == 0;
    };
    if (name == "token_embd.weight" || name == "output.weight") { *n = c.vocab; *k = c.hidden; return true; }
    if (name == "output_norm.weight") { *n = c.hidden; *k = 0; return true; }
    if (name.rfind("blk.", 0) != 0) return false;
    if (ends(".attn_norm.weight") || ends(".ffn_norm.weight")) { *n = c.hidden; *k = 0; return true; }
    if (ends(".attn_q_norm.weight") || ends(".attn_k_norm.weight")) { *n = c.head_dim; *k = 0; return true; }
    if (ends(".attn_q.weight")) { *n = qd; *k = c.hidden; return true; }
    if (ends(".attn_k.weight") || ends(".attn_v.weight")) { *n = kd; *k = c.hidden; return true; }
    if (ends(".attn_output.weight")) { *n = c.hidden; *k = qd; return true; }
    if (ends(".ffn_gate.weight") || ends(".ffn_up.weight")) { *n = c.ffn; *k = c.hidden; return true; }
    if (ends(".ffn_down.weight")) { *n = c.hidden; *k = c.ffn; return true; }
    if (c.n_expert) {  // stacked experts, [n_expert, out, in] in the file (reference: src/quantized_qwen3_moe.rs:556-571)
        if (ends(".ffn_gate_inp.weight")) { *n = (size_t)c.n_expert * c.hidden; *k = 0; return true; }
        if (ends(".ffn_gate_exps.weight") || ends(".ffn_up_exps.weight")) { *n = (size_t)c.n_expert * c.expert_ffn; *k = c.hidden; return true; }
        if (ends(".ffn_down_exps.weight")) { *n = (size_t)c.n_expert * c.hidden; *k = c.expert_ffn; return true; }
    }
    return false;
}

int model_mm(jq_model *m, const std::string &name, const float *x, float *y, size_t T, hipStream_t s) {
    auto it = m->q.find(name);
    if (it == m->q.end()) return fail("qwen3: missing tensor `%s`", name.c_str());
    const jq_weight *w = it->second;
    return dispatch_matmul(w->type, w->dev, w->row_bytes, x, y, T, w->k, w->n, s);
}

int model_vec(jq_model *m, const std::string &name, const float **out) {
    auto it = m->f.find(name);
    if (it == m->f.end()) return fail("qwen3: missing tensor `%s`", name.c_str());
    *out = it->second;
    return 0;
}

// Lays the named matrices (same type, same k) one after the other in a new allocation `key`, and
// replaces their entries in m->q by views of it.  Skipped when any is missing or the types differ.
// With `pair_rows` (two parts of equal shape) the rows alternate instead: row 2j of the fused matrix is
// row j of the first part, row 2j + 1 row j of the second, and the views stride over every other row.
int model_fuse(jq_model *m, const std::string &key, const std::vector<std::string> &names, bool pair_rows = false) {
    std::vector<jq_weight *> parts;
    for (const auto &nm : names) {
        auto it = m->q.find(nm);
        if (it == m->q.end() || !it->second->owns) return 0;
        parts.push_back(it->second);
    }
    size_t rows = 0, bytes = 0;
    for (auto *w : parts) {
        if (w->type != parts[0]->type || w->k != parts[0]->k) return 0;
        rows += w->n, bytes += w->nbytes;
    }
    pair_rows = pair_rows && parts.size() == 2 && parts[0]->n == parts[1]->n;
    const size_t rb = parts[0]->row_bytes;
    uint8_t *dev = nullptr;
    HIP_TRY(hipMalloc((void **)&dev, bytes));
    size_t off = 0;
    for (size_t i = 0; i < parts.size(); i++) {
        jq_weight *w = parts[i];
        hipError_t e = pair_rows ? hipMemcpy2D(dev + i * rb, 2 * rb, w->dev, rb, rb, w->n, hipMemcpyDeviceToDevice)
                                 : hipMemcpy(dev + off, w->dev, w->nbytes, hipMemcpyDeviceToDevice);
        if (e != hipSuccess) {
            (void)hipFree(dev);
            return fail("qwen3: fusing `%s` failed: %s", key.c_str(), hipGetErrorString(e));
        }
        off += w->nbytes;
    }
    jq_weight *whole = new jq_weight{parts[0]->type, rows, parts[0]->k, bytes, rb, dev, true};
    m->fused[key] = whole;
    if (pair_rows) m->paired.insert(key);
    off = 0;
    for (size_t i = 0; i < parts.size(); i++) {
        jq_weight *view = nullptr;
        if (pair_rows) {
            view = new jq_weight{whole->type, parts[i]->n, parts[i]->k, bytes - i * rb, 2 * rb, dev + i * rb, false};
        } else if (jq_view(whole, off, parts[i]->n, parts[i]->k, &view)) {
            return 1;
        }
        off += parts[i]->nbytes;
        jq_free(parts[i]);
        m->q[names[i]] = view;
    }
    return 0;
}

// The layer objects of a mixture-of-experts model that are not built yet (all of them at the first step).
int model_prepare_moe(jq_model *m) {
    const jq_qwen3_config &c = m->cfg;
    if (!c.n_expert) return 0;
    m->moe.resize(c.n_layer, nullptr);
    for (uint32_t l = 0; l < c.n_layer; l++) {
        if (m->moe[l]) continue;
        const std::string p = "blk." + std::to_string(l);
        auto r = m->router_host.find(p + ".ffn_gate_inp.weight");
        auto g = m->q.find(p + ".ffn_gate_exps.weight"), u = m->q.find(p + ".ffn_up_exps.weight"),
             d = m->q.find(p + ".ffn_down_exps.weight");
        if (r == m->router_host.end()) return fail("qwen3moe: missing tensor `%s.ffn_gate_inp.weight`", p.c_str());
        for (auto *it : {&g, &u, &d})
            if (*it == m->q.end()) return fail("qwen3moe: missing an expert tensor of `%s`", p.c_str());
        // softmax over all experts, top k, weights divided by their sum when norm_topk_prob
        // (reference: src/quantized_qwen3_moe.rs:424-436)
        jq_moe_config mc{};
        mc.n_expert = c.n_expert, mc.n_expert_used = c.n_expert_used, mc.hidden = c.hidden, mc.inter = c.expert_ffn;
        mc.gating = 0, mc.norm_topk = c.norm_topk_prob ? 1 : 0;
        if (jq_moe_create(&mc, r->second.data(), nullptr, g->second, u->second, d->second, nullptr, nullptr, nullptr, &m->moe[l]))
            return 1;
    }
    return 0;
}

int model_prepare_fused(jq_model *m) {
    if (model_prepare_moe(m)) return 1;
    if (m->fused_ready) return 0;
    const jq_qwen3_config &c = m->cfg;
    for (uint32_t l = 0; l < c.n_layer; l++) {
        const std::string p = "blk." + std::to_string(l);
        if (!m->fused.count(p + ".qkv")) {
            // q|k|v when all three share a type, else q|k (attn_v is often kept at more bits)
            auto q = m->q.find(p + ".attn_q.weight"), v = m->q.find(p + ".attn_v.weight");
            const bool with_v = q != m->q.end() && v != m->q.end() && q->second->type == v->second->type;
            if (model_fuse(m, p + ".qkv",
                           with_v ? std::vector<std::string>{p + ".attn_q.weight", p + ".attn_k.weight", p + ".attn_v.weight"}
                                  : std::vector<std::string>{p + ".attn_q.weight", p + ".attn_k.weight"}))
                return 1;
        }
        if (!c.n_expert && !m->fused.count(p + ".gate_up")) {
            // 4096-wide Q4_K rows: paired, for the launch that also applies SwiGLU
            auto g = m->q.find(p + ".ffn_gate.weight");
            const bool pair = g != m->q.end() && g->second->type == JQ_TYPE_Q4_K && g->second->k == 4096 &&
                              g->second->row_bytes == jq::QD_ROW && !getenv("JQ_NO_PAIRED_GATE_UP");
            if (model_fuse(m, p + ".gate_up", {p + ".ffn_gate.weight", p + ".ffn_up.weight"}, pair)) return 1;
        }
    }
    if (!m->cat) {
        const size_t widest = std::max<size_t>((size_t)(c.n_head + 2 * c.n_kv_head) * c.head_dim, 2 * (size_t)c.ffn);
        HIP_TRY(hipMalloc((void **)&m->cat, widest * sizeof(float)));
    }
    m->fused_ready = true;
    return 0;
}

unsigned grid_for(size_t total) { return (unsigned)std::min<size_t>((total + 255) / 256, 8192); }

// x_out = x + res; y = W rmsnorm(x_out) as one launch (hn_out also gets the normalised row when
// given).  False when no kernel has that form for this weight: the caller then runs the two steps.
// With `swiglu`, w pairs gate and up rows and y gets the w->n / 2 activations.
bool model_norm_mm(const jq_weight *w, const float *x, const float *res, const float *norm_w, float eps, float *x_out,
                   float *hn_out, float *y, bool swiglu, hipStream_t s) {
    static const char *off = getenv("JQ_NO_FUSED_NORM");
    if (off || w->type != JQ_TYPE_Q4_K) return false;
    const jq::QdNorm nm{res, norm_w, eps, x_out, hn_out};
    return dispatch_q4k_dot4(w->dev, w->row_bytes, x, y, w->k, w->n, s, &nm, swiglu) == 0;
}

int model_forward_dev(jq_model *m, uint32_t T, uint32_t pos, hipStream_t s) {
    const jq_qwen3_config &c = m->cfg;
    const int d = (int)c.head_dim, nh = (int)c.n_head, nkv = (int)c.n_kv_head, h = (int)c.hidden;
    auto emb = m->q.find("token_embd.weight");
    if (emb == m->q.end()) return fail("qwen3: missing tensor `token_embd.weight`");
    if (dispatch_decode(emb->second, m->ids, m->x, T, s)) return 1;
    // few query rows over a long cache: split the keys over the chip
    const bool split = T <= 8 && (d == 64 || d == 128 || d == 256);
    // the step's position for the kernels, and with split attention the rotary angles of its tokens
    hipLaunchKernelGGL(jq::rope_table, dim3(1), dim3(256), 0, s, m->pos, (int)pos, split ? (int)T : 0, d, c.rope_theta, m->rope_cs);
    const float sqrt_d = sqrtf((float)d);
    const int n_chunks = (int)((pos + T + jq::ATT_CHUNK - 1) / jq::ATT_CHUNK);
    const float *pending = nullptr;  // residual not yet added into x
    float *xc = m->x, *xo = m->x2;   // the residual stream, and where a fused norm + matmul launch writes its update
    for (uint32_t l = 0; l < c.n_layer; l++) {
        const std::string p = "blk." + std::to_string(l);
        const float *w_an, *w_fn, *w_qn, *w_kn;
        if (model_vec(m, p + ".attn_norm.weight", &w_an) || model_vec(m, p + ".ffn_norm.weight", &w_fn) ||
            model_vec(m, p + ".attn_q_norm.weight", &w_qn) || model_vec(m, p + ".attn_k_norm.weight", &w_kn))
            return 1;
        float *qp = m->qb, *kp = m->kb, *vp = m->vb;
        int q_stride = (int)(nh * d), k_stride = (int)(nkv * d), v_stride = (int)(nkv * d);  // floats from a token to the next
        auto fq = T == 1 ? m->fused.find(p + ".qkv") : m->fused.end();
        static const char *no_fused_prefill = getenv("JQ_NO_FUSED_QKV_PREFILL");
        // (the split attention kernel of steps up to 8 tokens reads q, k and v of a token as rows of their own)
        auto fqm = T > 1 && !split && !no_fused_prefill ? m->fused.find(p + ".qkv") : m->fused.end();
        bool v_fused = fq != m->fused.end() && fq->second->n == (size_t)(nh + 2 * nkv) * d;
        // single token: residual add, norm and q|k(|v) as one launch when the kernel has that form; an attn_v of
        // another format (Q6_K, Q8_0) rides in the same launch where its tiles fit beside the q|k workgroups
        bool normed = false;
        if (fq != m->fused.end() && !v_fused && fq->second->type == JQ_TYPE_Q4_K) {
            auto vw = m->q.find(p + ".attn_v.weight");
            if (vw != m->q.end() && vw->second->k == fq->second->k && vw->second->n == (size_t)nkv * d) {
                const jq_weight *w1 = fq->second, *w2 = vw->second;
                const jq::QdNorm nm{pending, w_an, c.rms_eps, xo, nullptr};
                const int rc = dispatch_q4k_norm_pair(w1->dev, w1->row_bytes, w1->n, w2->type, w2->dev, w2->row_bytes, w2->n, w1->k, xc,
                                                      m->cat, m->cat + w1->n, nm, s);
                if (rc > 0) return 1;
                if (rc == 0) normed = v_fused = true;
            }
        }
        if (!normed)
            normed = fq != m->fused.end() &&
                     model_norm_mm(fq->second, xc, pending, w_an, c.rms_eps, xo, v_fused ? nullptr : m->hn, m->cat, false, s);
        if (normed) std::swap(xc, xo);
        else hipLaunchKernelGGL(jq::rmsnorm_rows, dim3(T), dim3(1024), 0, s, xc, pending, w_an, c.rms_eps, m->hn, h);
        if (fq != m->fused.end()) {  // one launch for q|k(|v) of a single token
            const jq_weight *w = fq->second;
            if (!normed && dispatch_matmul(w->type, w->dev, w->row_bytes, m->hn, m->cat, 1, w->k, w->n, s)) return 1;
            qp = m->cat, kp = m->cat + (size_t)nh * d;
            if (v_fused) vp = kp + (size_t)nkv * d;
            else if (model_mm(m, p + ".attn_v.weight", m->hn, m->vb, T, s)) return 1;
        } else if (fqm != m->fused.end()) {
            // several tokens: q|k(|v) as one product, whose rows hold a token's q, k (and v) heads side by side
            const jq_weight *w = fqm->second;
            if (dispatch_matmul(w->type, w->dev, w->row_bytes, m->hn, m->qb, T, w->k, w->n, s)) return 1;
            q_stride = k_stride = (int)w->n;
            kp = m->qb + (size_t)nh * d;
            if (w->n == (size_t)(nh + 2 * nkv) * d) vp = kp + (size_t)nkv * d, v_stride = (int)w->n;
            else if (model_mm(m, p + ".attn_v.weight", m->hn, m->vb, T, s)) return 1;
        } else if (model_mm(m, p + ".attn_q.weight", m->hn, m->qb, T, s) ||
                   model_mm(m, p + ".attn_k.weight", m->hn, m->kb, T, s) ||
                   model_mm(m, p + ".attn_v.weight", m->hn, m->vb, T, s)) {
            return 1;
        }
        if (split) {  // head norm, rotation and cache writes happen inside the attention kernel
            const int n_tri = (int)(T * nkv * n_chunks);
#define JQ_ATT_SPLIT(D)                                                                                          \
    hipLaunchKernelGGL(jq::attention_split<D>, dim3(8 * (nh / nkv) * ((n_tri + 7) / 8)), dim3(256), 0, s, nh, nkv, \
                       n_chunks, n_tri, (int)pos, (int)c.n_ctx, qp, kp, vp, m->kc[l], m->vc[l], w_qn, w_kn,         \
                       m->rope_cs, m->part, c.rms_eps, sqrt_d)
            if (d == 64) JQ_ATT_SPLIT(64);
            else if (d == 128) JQ_ATT_SPLIT(128);
            else JQ_ATT_SPLIT(256);
#undef JQ_ATT_SPLIT
            hipLaunchKernelGGL(jq::attention_merge, dim3(T * nh), dim3(128), 2 * n_chunks * sizeof(float), s, m->part, m->att, d,
                               n_chunks);
        } else {
            hipLaunchKernelGGL(jq::qkv_norm_rope_cache, dim3(T * (nh + 2 * nkv)), dim3(64), 0, s, qp, kp, vp, w_qn, w_kn,
                               c.rms_eps, nh, nkv, d, m->pos, c.rope_theta, m->kc[l], m->vc[l], (int)c.n_ctx, q_stride,
                               k_stride, v_stride);
            // head dimension 128 and 1, 2, 4 or 8 query heads a KV head: tiles of 16 tokens on the f32 matrix cores
            static const char *no_tiles = getenv("JQ_NO_ATTENTION_TILES");
            const int gq = nh / nkv;
            const dim3 tgrid((unsigned)((T + 15) / 16), (unsigned)nkv);
#define JQ_ATT_TILES(GQ, KS)                                                                                        \
    hipLaunchKernelGGL((jq::attention_tiles<128, GQ, KS>), tgrid, dim3(64 * GQ * KS), 0, s, qp, m->kc[l], m->vc[l],   \
                       m->att, (int)T, nh, m->pos, (int)c.n_ctx, sqrt_d, q_stride)
            // two key splits a workgroup once the last tokens walk 8 key tiles or more (up to 4 query heads a KV
            // head: the merge of 8 would not fit the static LDS)
            static const char *no_split_env = getenv("JQ_ATTENTION_TILES_NO_KEY_SPLIT");
            const bool ksplit = !no_split_env && pos + T >= 128;
            if (no_tiles || d != 128 || (gq != 1 && gq != 2 && gq != 4 && gq != 8)) {
                size_t sm = ((size_t)d + jq::AR_CHUNK + 16) * sizeof(float);
                hipLaunchKernelGGL(jq::attention_rows, dim3(T * nh), dim3(256), sm, s, qp, m->kc[l], m->vc[l], m->att, nh,
                                   nkv, d, m->pos, (int)c.n_ctx, sqrt_d, q_stride);
            } else if (gq == 1 && ksplit) JQ_ATT_TILES(1, 2);
            else if (gq == 1) JQ_ATT_TILES(1, 1);
            else if (gq == 2 && ksplit) JQ_ATT_TILES(2, 2);
            else if (gq == 2) JQ_ATT_TILES(2, 1);
            else if (gq == 4 && ksplit) JQ_ATT_TILES(4, 2);
            else if (gq == 4) JQ_ATT_TILES(4, 1);
            else JQ_ATT_TILES(8, 1);
#undef JQ_ATT_TILES
        }
        if (model_mm(m, p + ".attn_output.weight", m->att, m->proj, T, s)) return 1;
        if (c.n_expert) {
            // x + moe(norm(x)) (reference: src/quantized_qwen3_moe.rs:806-812)
            jq_moe *moe = m->moe[l];
            if (m->moe_scratch_at >= 0 && m->moe_scratch_at != (int)l && m->moe[m->moe_scratch_at])
                moe_swap_scratch(moe, m->moe[m->moe_scratch_at]);
            m->moe_scratch_at = (int)l;
            // (the norm: inside the router launch for a single token, else a launch of its own in place)
            MoePreNorm pre{jq::MoePreNormArgs{xc, m->proj, w_fn, c.rms_eps, xo, m->hn}, false};
            {
                std::lock_guard<std::mutex> lock(moe->mu);
                if (moe_reserve(moe, T) || moe_forward_dev(moe, T, m->hn, m->proj, s, &pre)) return 1;
            }
            if (pre.fused) std::swap(xc, xo);
            pending = m->proj;
            continue;
        }
        const float *gp = m->g, *up = m->u;
        auto fg = T == 1 ? m->fused.find(p + ".gate_up") : m->fused.end();
        const bool paired = fg != m->fused.end() && m->paired.count(fg->first);  // gate and up rows alternate
        bool activated = false;  // m->mid already holds silu(gate) * up
        bool down_done = false;  // m->proj already holds the down projection
        const bool normed2 = fg != m->fused.end() && model_norm_mm(fg->second, xc, m->proj, w_fn, c.rms_eps, xo, nullptr,
                                                                   paired ? m->mid : m->cat, paired, s);
        if (normed2) std::swap(xc, xo), activated = paired;
        else hipLaunchKernelGGL(jq::rmsnorm_rows, dim3(T), dim3(1024), 0, s, xc, m->proj, w_fn, c.rms_eps, m->hn, h);
        // many tokens over a paired gate|up matrix: one product with twice the rows (768 GEMM tiles at Qwen3-8B's
        // sizes fill the 256 compute units three times over; two products of 384 tiles leave half of them idle
        // in their second rounds), then SwiGLU over the alternating results
        static const char *no_pair_gemm = getenv("JQ_NO_PAIRED_PREFILL");
        auto fgm = T > 1 && !no_pair_gemm ? m->fused.find(p + ".gate_up") : m->fused.end();
        if (fgm != m->fused.end() && !m->paired.count(fgm->first)) fgm = m->fused.end();
        if (fg != m->fused.end()) {
            const jq_weight *w = fg->second;
            if (!normed2 && dispatch_matmul(w->type, w->dev, w->row_bytes, m->hn, m->cat, 1, w->k, w->n, s)) return 1;
            gp = m->cat, up = m->cat + c.ffn;
        } else if (fgm != m->fused.end()) {
            const jq_weight *w = fgm->second;
            if (dispatch_matmul(w->type, w->dev, w->row_bytes, m->hn, m->g, T, w->k, w->n, s)) return 1;
            // many rows into a Q4_K or Q6_K down projection: the int8 GEMM's activation preparation applies
            // SwiGLU to the pairs as it reads them
            auto dn = m->q.find(p + ".ffn_down.weight");
            static const char *no_fused_swiglu = getenv("JQ_NO_SWIGLU_IN_PREP");
            if (dn != m->q.end() && !no_fused_swiglu && dn->second->k == c.ffn) {
                const jq_weight *wd = dn->second;
                int rc = -1;
                if (wd->type == JQ_TYPE_Q4_K)
                    rc = dispatch_gemm_i8<jq::QiQ4K>(wd->dev, wd->row_bytes, m->g, m->proj, T, wd->k, wd->n, s, "q4k_gemm_i8",
                                                     "q4k_gemm_i8+splitk", true);
                else if (wd->type == JQ_TYPE_Q6_K)
                    rc = dispatch_gemm_i8<jq::QiQ6K>(wd->dev, wd->row_bytes, m->g, m->proj, T, wd->k, wd->n, s, "q6k_gemm_i8",
                                                     "q6k_gemm_i8+splitk", true);
                if (rc > 0) return 1;
                down_done = rc == 0;
            }
            if (!down_done)
                hipLaunchKernelGGL(jq::swiglu_pairs, dim3(grid_for((size_t)T * c.ffn)), dim3(256), 0, s, m->g, m->mid, (size_t)T * c.ffn);
            activated = true;
        } else if (model_mm(m, p + ".ffn_gate.weight", m->hn, m->g, T, s) ||
                   model_mm(m, p + ".ffn_up.weight", m->hn, m->u, T, s)) {
            return 1;
        }
        if (activated) {
        } else if (paired) {
            hipLaunchKernelGGL(jq::swiglu_pairs, dim3(grid_for((size_t)c.ffn)), dim3(256), 0, s, m->cat, m->mid, (size_t)c.ffn);
        } else {
            hipLaunchKernelGGL(jq::swiglu_rows, dim3(grid_for((size_t)T * c.ffn)), dim3(256), 0, s, gp, up, m->mid,
                               (size_t)T * c.ffn, 0.0f);
        }
        if (!down_done && model_mm(m, p + ".ffn_down.weight", m->mid, m->proj, T, s)) return 1;
        pending = m->proj;
    }
    const float *w_on;
    if (model_vec(m, "output_norm.weight", &w_on)) return 1;
    // logits only for the last position (reference: src/quantized_qwen3_moe.rs:816-818)
    const size_t last = (size_t)(T - 1) * h;
    hipLaunchKernelGGL(jq::rmsnorm_rows, dim3(1), dim3(1024), 0, s, xc + last, pending ? pending + last : nullptr, w_on,
                       c.rms_eps, m->hn, h);
    // tie_word_embeddings conversions ship no output head (src/quantized_qwen3_moe.rs:739-743)
    const char *head = m->q.count("output.weight") ? "output.weight" : "token_embd.weight";
    if (model_mm(m, head, m->hn, m->logits, 1, s)) return 1;
    HIP_TRY(hipGetLastError());
    return 0;
}

}  // namespace

extern "C" {

int jq_qwen3_create(const jq_qwen3_config *cfg, jq_model **out) {
    if (!out) return fail("jq_qwen3_create: out is null");
    *out = nullptr;
    if (!cfg) return fail("jq_qwen3_create: cfg is null");
    const jq_qwen3_config &c = *cfg;
    if (!c.n_layer || !c.hidden || !c.n_head || !c.n_kv_head || !c.head_dim || !c.vocab || !c.n_ctx ||
        (!c.ffn && !c.n_expert))
        return fail("qwen3: zero in configuration");
    // reference: src/quantized_qwen3_moe.rs:122-129
    if (c.n_expert && (c.n_expert_used == 0 || c.n_expert_used > c.n_expert))
        return fail("qwen3moe: expert_used_count %u must be in 1..=expert_count %u", c.n_expert_used, c.n_expert);
    if (c.n_expert && c.expert_ffn == 0) return fail("qwen3moe: expert_feed_forward_length must be positive");
    if (c.n_head % c.n_kv_head != 0) return fail("qwen3: %u query heads over %u kv heads", c.n_head, c.n_kv_head);
    if (c.head_dim % 8 != 0 || c.hidden % 4 != 0 || c.ffn % 4 != 0) return fail("qwen3: dimensions must be multiples of 4/8");
    if (c.head_dim > (uint32_t)jq::AR_MAX_D) return fail("qwen3: head_dim %u exceeds %d", c.head_dim, jq::AR_MAX_D);
    if (ensure_init()) return 1;
    jq_model *m = new jq_model;
    m->cfg = c;
    size_t per = (size_t)c.n_kv_head * c.n_ctx * c.head_dim * sizeof(float);
    for (uint32_t l = 0; l < c.n_layer; l++) {
        float *k = nullptr, *v = nullptr;
        if (hipMalloc((void **)&k, per) != hipSuccess || hipMalloc((void **)&v, per) != hipSuccess) {
            if (k) (void)hipFree(k);
            jq_qwen3_free(m);
            return fail("qwen3: KV cache allocation failed (%zu bytes per layer)", 2 * per);
        }
        m->kc.push_back(k);
        m->vc.push_back(v);
    }
    const size_t part_floats = (size_t)8 * c.n_head * ((c.n_ctx + jq::ATT_CHUNK - 1) / jq::ATT_CHUNK) * (c.head_dim + 2);
    if (hipMalloc((void **)&m->logits, c.vocab * sizeof(float)) != hipSuccess ||
        hipMalloc((void **)&m->pick, sizeof(uint32_t)) != hipSuccess ||
        hipMalloc((void **)&m->pick_v, jq::ARGMAX_PARTS * sizeof(float)) != hipSuccess ||
        hipMalloc((void **)&m->pick_i, jq::ARGMAX_PARTS * sizeof(int)) != hipSuccess ||
        hipMalloc((void **)&m->pos, sizeof(int)) != hipSuccess ||
        hipMalloc((void **)&m->part, part_floats * sizeof(float)) != hipSuccess ||
        hipMalloc((void **)&m->rope_cs, (size_t)8 * (c.head_dim / 2) * sizeof(float2)) != hipSuccess) {
        jq_qwen3_free(m);
        return fail("qwen3: logits allocation failed");
    }
    *out = m;
    return 0;
}

void jq_qwen3_free(jq_model *m) {
    if (!m) return;
    model_free_scratch(m);
    for (jq_moe *e : m->moe) jq_moe_free(e);
    for (auto &kv : m->q) jq_free(kv.second);
    for (auto &kv : m->fused) jq_free(kv.second);
    for (auto *w : m->retired) jq_free(w);
    if (m->cat) (void)hipFree(m->cat);
    for (auto &kv : m->f) (void)hipFree(kv.second);
    for (float *p : m->kc) (void)hipFree(p);
    for (float *p : m->vc) (void)hipFree(p);
    if (m->logits) (void)hipFree(m->logits);
    if (m->pick) (void)hipFree(m->pick);
    if (m->pick_v) (void)hipFree(m->pick_v);
    if (m->pick_i) (void)hipFree(m->pick_i);
    if (m->pos) (void)hipFree(m->pos);
    if (m->part) (void)hipFree(m->part);
    if (m->rope_cs) (void)hipFree(m->rope_cs);
    delete m;
}

int jq_qwen3_set_tensor(jq_model *m, const char *name, uint32_t ggml_type, const void *data, size_t nbytes) {
    if (!m || !name || !data) return fail("jq_qwen3_set_tensor: null argument");
    size_t n, k;
    if (!qwen3_shape(m->cfg, name, &n, &k)) return fail("qwen3: unknown tensor `%s`", name);
    std::lock_guard<std::mutex> lock(m->mu);
    const std::string nm = name;
    const size_t dot = nm.find('.', 4);
    const bool in_layer = nm.rfind("blk.", 0) == 0 && dot != std::string::npos;
    const std::string role = in_layer ? nm.substr(dot) : std::string();
    if (role == ".ffn_gate_inp.weight" || role == ".ffn_gate_exps.weight" || role == ".ffn_up_exps.weight" ||
        role == ".ffn_down_exps.weight") {
        // the layer object is rebuilt from the new tensors at the next step
        const size_t l = (size_t)atoll(nm.c_str() + 4);
        if (l < m->moe.size() && m->moe[l]) {
            if (m->moe_scratch_at == (int)l) m->moe_scratch_at = -1;  // its scratch goes with it
            jq_moe_free(m->moe[l]);
            m->moe[l] = nullptr;
        }
    }
    if (role == ".ffn_gate_inp.weight") {
        // the router is read as f32 whatever the file holds (reference: src/quantized_qwen3_moe.rs:197-199, :654-657)
        std::vector<float> host(n);
        if (ggml_type == 0 && nbytes == n * sizeof(float)) {
            memcpy(host.data(), data, nbytes);
        } else if (ggml_type == 1 && nbytes == n * sizeof(uint16_t)) {
            const uint16_t *hsrc = (const uint16_t *)data;
            for (size_t i = 0; i < n; i++) {
                _Float16 hv;
                memcpy(&hv, hsrc + i, sizeof hv);
                host[i] = (float)hv;
            }
        } else {
            return fail("qwen3moe: `%s` must be F32 or F16 with %zu values (type %u, %zu bytes)", name, n, ggml_type, nbytes);
        }
        m->router_host[nm] = std::move(host);
        return 0;
    }
    if (k == 0) {
        if (ggml_type != 0) return fail("qwen3: `%s` must be F32", name);
        if (nbytes != n * sizeof(float)) return fail("qwen3: `%s` holds %zu bytes, expected %zu", name, nbytes, n * sizeof(float));
        float *dev = nullptr;
        HIP_TRY(hipMalloc((void **)&dev, nbytes));
        hipError_t e = hipMemcpy(dev, data, nbytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            (void)hipFree(dev);
            return fail("qwen3: upload of `%s` failed: %s", name, hipGetErrorString(e));
        }
        auto old = m->f.find(name);
        if (old != m->f.end()) (void)hipFree(old->second);
        m->f[name] = dev;
        return 0;
    }
    jq_weight *w = nullptr;
    if (jq_upload(ggml_type, data, nbytes, n, k, 0, &w)) return 1;
    auto old = m->q.find(name);
    if (old != m->q.end()) jq_free(old->second);
    m->q[name] = w;
    // a replaced part: the fused copy it belonged to is retired (the other parts' views keep pointing
    // into it) and that group runs as separate launches from now on
    if (in_layer) {
        const std::string layer = nm.substr(0, dot);
        const char *key = (role == ".attn_q.weight" || role == ".attn_k.weight" || role == ".attn_v.weight") ? ".qkv"
                          : (role == ".ffn_gate.weight" || role == ".ffn_up.weight")                         ? ".gate_up"
                                                                                                             : nullptr;
        if (key) {
            auto it = m->fused.find(layer + key);
            if (it != m->fused.end()) {
                m->retired.push_back(it->second);
                m->paired.erase(it->first);
                m->fused.erase(it);
            }
        }
    }
    return 0;
}

int jq_qwen3_forward(jq_model *m, const uint32_t *tokens, uint32_t n_tokens, uint32_t pos, float *logits,
                     int logits_on_device, void *stream) {
    if (!m || !tokens) return fail("jq_qwen3_forward: null argument");
    if (n_tokens == 0) return fail("qwen3: forward needs at least one token");
    std::lock_guard<std::mutex> lock(m->mu);
    // the KV-cache contract of the plugin boundary (reference: crates/joshua-mock-npu/src/lib.rs:89-95)
    if (pos != m->n_past) return fail("qwen3: pos %u does not match the %u tokens fed so far", pos, m->n_past);
    if ((uint64_t)pos + n_tokens > m->cfg.n_ctx)
        return fail("qwen3: %u + %u tokens exceed the context of %u", pos, n_tokens, m->cfg.n_ctx);
    for (uint32_t i = 0; i < n_tokens; i++)
        if (tokens[i] >= m->cfg.vocab) return fail("embedding id %u is out of range for %u rows", tokens[i], m->cfg.vocab);
    hipStream_t s = (hipStream_t)stream;
    if (model_reserve(m, n_tokens)) return 1;
    if (model_prepare_fused(m)) return 1;  // first step only: q|k(|v) and gate|up as single matrices
    HIP_TRY(hipMemcpyAsync(m->ids, tokens, n_tokens * sizeof(uint32_t), hipMemcpyHostToDevice, s));
    if (model_forward_dev(m, n_tokens, pos, s)) return 1;
    m->n_past = pos + n_tokens;
    if (logits) {
        HIP_TRY(hipMemcpyAsync(logits, m->logits, m->cfg.vocab * sizeof(float),
                               logits_on_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost, s));
        if (!logits_on_device) HIP_TRY(hipStreamSynchronize(s));
    }
    return 0;
}

int jq_qwen3_greedy(jq_model *m, uint32_t *token, void *stream) {
    if (!m || !token) return fail("jq_qwen3_greedy: null argument");
    hipStream_t s = (hipStream_t)stream;
    std::lock_guard<std::mutex> lock(m->mu);
    hipLaunchKernelGGL(jq::argmax_last_parts, dim3(jq::ARGMAX_PARTS), dim3(256), 0, s, m->logits, (int)m->cfg.vocab,
                       m->pick_v, m->pick_i);
    hipLaunchKernelGGL(jq::argmax_last_merge, dim3(1), dim3(jq::ARGMAX_PARTS), 0, s, m->pick_v, m->pick_i, m->pick);
    HIP_TRY(hipMemcpyAsync(token, m->pick, sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    HIP_TRY(hipStreamSynchronize(s));
    return 0;
}

int jq_qwen3_get_config(const jq_model *m, jq_qwen3_config *out) {
    if (!m || !out) return fail("jq_qwen3_get_config: null argument");
    *out = m->cfg;
    return 0;
}

int jq_qwen3_reset(jq_model *m) {
    if (!m) return fail("jq_qwen3_reset: model is null");
    std::lock_guard<std::mutex> lock(m->mu);
    m->n_past = 0;
    return 0;
}

}  // extern "C"

// ---- GGUF files and the model-level plugin boundary ------------------------------------------

#include "gguf.hpp"

struct jq_gguf {
    std::unique_ptr<jq::Gguf> g;
};

namespace {

int gguf_wrap(std::unique_ptr<jq::Gguf> g, const std::string &err, jq_gguf **out) {
    if (!g) return fail("%s", err.c_str());
    *out = new jq_gguf{std::move(g)};
    return 0;
}

// Every tensor the graph reads is installed, or the name of the first one that is not.
int model_check_complete(jq_model *m) {
    std::vector<std::string> names = {"token_embd.weight", "output_norm.weight", "output.weight"};
    const bool moe = m->cfg.n_expert != 0;
    for (uint32_t l = 0; l < m->cfg.n_layer; l++) {
        for (const char *role : {"attn_norm", "attn_q", "attn_k", "attn_v", "attn_q_norm", "attn_k_norm", "attn_output", "ffn_norm"})
            names.push_back("blk." + std::to_string(l) + "." + role + ".weight");
        for (const char *role : {moe ? "ffn_gate_inp" : "ffn_gate", moe ? "ffn_gate_exps" : "ffn_up", moe ? "ffn_up_exps" : "ffn_down"})
            names.push_back("blk." + std::to_string(l) + "." + role + ".weight");
        if (moe) names.push_back("blk." + std::to_string(l) + ".ffn_down_exps.weight");
    }
    for (const auto &nm : names)
        if (!m->q.count(nm) && !m->f.count(nm) && !m->router_host.count(nm))
            return fail("%s: missing tensor `%s`", moe ? "qwen3moe" : "qwen3", nm.c_str());
    return 0;
}

// Configuration of a dense qwen3 file from its metadata, with the reference loader's rules
// (reference: src/quantized_qwen3_moe.rs:90-147): attention.key_length wins over
// embedding_length / head_count, rope.freq_base defaults to 10000, head_count must be a multiple
// of head_count_kv, head_dim must be positive and even.
int qwen3_config_from_gguf(const jq::Gguf &g, uint32_t n_ctx, jq_qwen3_config *c) {
    const std::string *arch = g.meta_str("general.architecture");
    if (!arch || (*arch != "qwen3" && *arch != "qwen3moe"))
        return fail("qwen3: general.architecture is `%s`, expected `qwen3` or `qwen3moe`", arch ? arch->c_str() : "(missing)");
    const std::string a = *arch;
    const bool moe = a == "qwen3moe";
    auto need_u32 = [&](const char *key, uint32_t *v) {
        if (g.meta_u32(a + "." + key, v)) return 0;
        return fail("%s: missing GGUF metadata key `%s.%s`", a.c_str(), a.c_str(), key);
    };
    uint32_t context_length = 0, key_length = 0;
    if (need_u32("attention.head_count", &c->n_head) || need_u32("attention.head_count_kv", &c->n_kv_head) ||
        need_u32("block_count", &c->n_layer) || need_u32("embedding_length", &c->hidden) ||
        need_u32("context_length", &context_length))
        return 1;
    if (!g.meta_f32(a + ".attention.layer_norm_rms_epsilon", &c->rms_eps))
        return fail("%s: missing GGUF metadata key `%s.attention.layer_norm_rms_epsilon`", a.c_str(), a.c_str());
    if (c->n_head == 0) return fail("%s: head_count is zero", a.c_str());
    c->head_dim = g.meta_u32(a + ".attention.key_length", &key_length) ? key_length : c->hidden / c->n_head;
    if (c->head_dim == 0 || c->head_dim % 2 != 0)
        return fail("%s: invalid head_dim %u (must be a positive even number)", a.c_str(), c->head_dim);
    if (c->n_kv_head == 0 || c->n_head % c->n_kv_head != 0)
        return fail("%s: head_count %u must be a multiple of head_count_kv %u", a.c_str(), c->n_head, c->n_kv_head);
    if (!g.meta_f32(a + ".rope.freq_base", &c->rope_theta)) c->rope_theta = 10000.0f;
    if (moe) {
        // reference: src/quantized_qwen3_moe.rs:119-134 (every layer's feed-forward block is a mixture of experts)
        if (need_u32("expert_count", &c->n_expert) || need_u32("expert_used_count", &c->n_expert_used) ||
            need_u32("expert_feed_forward_length", &c->expert_ffn))
            return 1;
        if (c->n_expert_used == 0 || c->n_expert_used > c->n_expert)
            return fail("qwen3moe: expert_used_count %u must be in 1..=expert_count %u", c->n_expert_used, c->n_expert);
        if (c->expert_ffn == 0) return fail("qwen3moe: expert_feed_forward_length must be positive");
        bool norm = true;
        if (!g.meta_bool("qwen3moe.attention.norm_topk_prob", &norm)) norm = true;
        c->norm_topk_prob = norm ? 1 : 0;
        c->ffn = 0;
    }
    // the two sizes the metadata may leave out are read off the tensors
    const jq::GgufTensor *emb = g.tensor("token_embd.weight");
    if (!emb || emb->dims.size() != 2) return fail("qwen3: missing tensor `token_embd.weight`");
    c->vocab = (uint32_t)emb->dims[0];
    if (!moe && !g.meta_u32("qwen3.feed_forward_length", &c->ffn)) {
        const jq::GgufTensor *gate = g.tensor("blk.0.ffn_gate.weight");
        if (!gate || gate->dims.size() != 2) return fail("qwen3: missing GGUF metadata key `qwen3.feed_forward_length`");
        c->ffn = (uint32_t)gate->dims[0];
    }
    c->n_ctx = n_ctx ? n_ctx : context_length;
    return 0;
}

}  // namespace

extern "C" {

int jq_type_size_bytes(uint32_t ggml_type, size_t elems, size_t *bytes) {
    uint64_t b;
    if (!bytes) return fail("jq_type_size_bytes: bytes is null");
    if (!jq::gguf_type_size_bytes(ggml_type, elems, &b))
        return fail("type id %u with %zu elements has no known size", ggml_type, elems);
    *bytes = (size_t)b;
    return 0;
}

int jq_gguf_open(const char *path, jq_gguf **out) {
    if (!path || !out) return fail("jq_gguf_open: null argument");
    *out = nullptr;
    std::string err;
    auto g = jq::gguf_open(path, &err);
    return gguf_wrap(std::move(g), err, out);
}

int jq_gguf_parse(const void *bytes, size_t len, jq_gguf **out) {
    if (!bytes || !out) return fail("jq_gguf_parse: null argument");
    *out = nullptr;
    std::vector<uint8_t> copy((const uint8_t *)bytes, (const uint8_t *)bytes + len);
    std::string err;
    auto g = jq::gguf_parse(copy.data(), copy.size(), &err);
    if (g) {
        g->owned = std::move(copy);  // moving a vector keeps its storage, so g->base stays valid
        g->base = g->owned.data();
    }
    return gguf_wrap(std::move(g), err, out);
}

void jq_gguf_close(jq_gguf *g) { delete g; }

uint32_t jq_gguf_version(const jq_gguf *g) { return g ? g->g->version : 0; }
uint64_t jq_gguf_tensor_data_offset(const jq_gguf *g) { return g ? g->g->tensor_data_offset : 0; }
size_t jq_gguf_tensor_count(const jq_gguf *g) { return g ? g->g->tensors.size() : 0; }
size_t jq_gguf_metadata_count(const jq_gguf *g) { return g ? g->g->metadata.size() : 0; }

int jq_gguf_tensor_at(const jq_gguf *g, size_t index, const char **name, uint32_t *ggml_type, uint32_t *n_dims,
                      uint64_t *dims, uint64_t *offset) {
    if (!g) return fail("jq_gguf_tensor_at: file is null");
    if (index >= g->g->tensors.size()) return fail("GGUF: tensor index %zu of %zu", index, g->g->tensors.size());
    const jq::GgufTensor &t = g->g->tensors[index];
    if (name) *name = t.name.c_str();
    if (ggml_type) *ggml_type = t.dtype;
    if (n_dims) *n_dims = (uint32_t)t.dims.size();
    if (dims)
        for (size_t d = 0; d < t.dims.size(); d++) dims[d] = t.dims[d];
    if (offset) *offset = t.offset;
    return 0;
}

int jq_gguf_find_tensor(const jq_gguf *g, const char *name, size_t *index) {
    if (!g || !name || !index) return fail("jq_gguf_find_tensor: null argument");
    auto it = g->g->by_name.find(name);
    if (it == g->g->by_name.end()) return fail("GGUF: no tensor `%s`", name);
    *index = it->second;
    return 0;
}

int jq_gguf_tensor_bytes(const jq_gguf *g, size_t index, const void **data, size_t *nbytes) {
    if (!g || !data || !nbytes) return fail("jq_gguf_tensor_bytes: null argument");
    if (index >= g->g->tensors.size()) return fail("GGUF: tensor index %zu of %zu", index, g->g->tensors.size());
    const uint8_t *p;
    uint64_t n;
    std::string err;
    if (!g->g->tensor_bytes(g->g->tensors[index], &p, &n, &err)) return fail("GGUF: %s", err.c_str());
    *data = p;
    *nbytes = (size_t)n;
    return 0;
}

int jq_gguf_meta_u32(const jq_gguf *g, const char *key, uint32_t *out) {
    if (!g || !key || !out) return fail("jq_gguf_meta_u32: null argument");
    return g->g->meta_u32(key, out) ? 0 : fail("GGUF: no unsigned 32-bit value under `%s`", key);
}

int jq_gguf_meta_f32(const jq_gguf *g, const char *key, float *out) {
    if (!g || !key || !out) return fail("jq_gguf_meta_f32: null argument");
    return g->g->meta_f32(key, out) ? 0 : fail("GGUF: no f32 value under `%s`", key);
}

int jq_gguf_meta_bool(const jq_gguf *g, const char *key, int *out) {
    if (!g || !key || !out) return fail("jq_gguf_meta_bool: null argument");
    bool b;
    if (!g->g->meta_bool(key, &b)) return fail("GGUF: no bool value under `%s`", key);
    *out = b;
    return 0;
}

int jq_gguf_meta_str(const jq_gguf *g, const char *key, const char **out, size_t *len) {
    if (!g || !key || !out) return fail("jq_gguf_meta_str: null argument");
    const std::string *s = g->g->meta_str(key);
    if (!s) return fail("GGUF: no string value under `%s`", key);
    *out = s->c_str();
    if (len) *len = s->size();
    return 0;
}

int jq_gguf_meta_array_len(const jq_gguf *g, const char *key, size_t *len) {
    if (!g || !key || !len) return fail("jq_gguf_meta_array_len: null argument");
    const jq::GgufValue *v = g->g->find(key);
    if (!v || v->type != 9) return fail("GGUF: no array under `%s`", key);
    *len = v->items.size();
    return 0;
}

int jq_gguf_upload(const jq_gguf *g, const char *name, jq_weight **out) {
    if (!g || !name || !out) return fail("jq_gguf_upload: null argument");
    *out = nullptr;
    const jq::GgufTensor *t = g->g->tensor(name);
    if (!t) return fail("GGUF: no tensor `%s`", name);
    if (t->dims.size() < 2) return fail("GGUF: tensor `%s` has %zu dimensions, a matrix needs 2", name, t->dims.size());
    const uint8_t *p;
    uint64_t nbytes;
    std::string err;
    if (!g->g->tensor_bytes(*t, &p, &nbytes, &err)) return fail("GGUF: %s", err.c_str());
    size_t k = (size_t)t->dims.back(), n = (size_t)(t->elem_count() / (k ? k : 1));
    return jq_upload(t->dtype, p, (size_t)nbytes, n, k, 0, out);
}

int jq_qwen3_load_gguf(const char *path, uint32_t n_ctx, jq_model **out) {
    if (!path || !out) return fail("jq_qwen3_load_gguf: null argument");
    *out = nullptr;
    std::string err;
    auto g = jq::gguf_open(path, &err);
    if (!g) return fail("%s", err.c_str());
    jq_qwen3_config cfg{};
    if (qwen3_config_from_gguf(*g, n_ctx, &cfg)) return 1;
    jq_model *m = nullptr;
    if (jq_qwen3_create(&cfg, &m)) return 1;
    bool have_output = false;
    for (const jq::GgufTensor &t : g->tensors) {
        size_t n, k;
        if (!qwen3_shape(cfg, t.name, &n, &k)) continue;  // rope tables and the like
        const uint8_t *p;
        uint64_t nbytes;
        if (!g->tensor_bytes(t, &p, &nbytes, &err)) {
            jq_qwen3_free(m);
            return fail("GGUF: %s", err.c_str());
        }
        bool shape_ok = k == 0 ? (t.dims.size() == 1 && t.dims[0] == n)
                               : (t.dims.size() == 2 && t.dims[0] == n && t.dims[1] == k);
        const bool router = t.name.size() > 20 && t.name.compare(t.name.size() - 20, 20, ".ffn_gate_inp.weight") == 0;
        const bool stacked = t.name.find("_exps.weight") != std::string::npos;
        if (router) shape_ok = t.dims.size() == 2 && t.dims[0] == cfg.n_expert && t.dims[1] == cfg.hidden;
        if (stacked) {
            if (t.dims.size() != 3 || t.dims[0] != cfg.n_expert) {
                jq_qwen3_free(m);
                return fail("qwen3moe: expected expert tensor `%s` shaped [n_expert, out, in]", t.name.c_str());
            }
            shape_ok = t.dims[0] * t.dims[1] == n && t.dims[2] == k;
        }
        if (!shape_ok) {
            jq_qwen3_free(m);
            return fail("qwen3: tensor `%s` does not have the shape the metadata implies", t.name.c_str());
        }
        if (jq_qwen3_set_tensor(m, t.name.c_str(), t.dtype, p, (size_t)nbytes)) {
            jq_qwen3_free(m);
            return 1;
        }
        have_output |= t.name == "output.weight";
    }
    if (!have_output) {
        // conversions with tied embeddings ship no output head
        // (reference: src/quantized_qwen3_moe.rs:739-743)
        const jq::GgufTensor *emb = g->tensor("token_embd.weight");
        const uint8_t *p;
        uint64_t nbytes;
        if (!emb || !g->tensor_bytes(*emb, &p, &nbytes, &err) ||
            jq_qwen3_set_tensor(m, "output.weight", emb->dtype, p, (size_t)nbytes)) {
            jq_qwen3_free(m);
            return emb ? 1 : fail("qwen3: missing tensor `token_embd.weight`");
        }
    }
    if (model_check_complete(m)) {
        jq_qwen3_free(m);
        return 1;
    }
    *out = m;
    return 0;
}

// The four symbols the reference engine binds when it loads a backend as a shared library
// (reference: src/npu/mod.rs:32-50 contract, src/npu/vendor.rs:17-20 signatures, :49-56 symbol
// check, :95-121 init; crates/joshua-mock-npu/src/lib.rs:41-131 return codes of the model plugin).
int32_t joshua_npu_init(const char *model_path, uint32_t n_ctx, uint32_t *out_vocab, void **out_handle) {
    if (!model_path || !out_vocab || !out_handle) return -1;
    *out_handle = nullptr;
    jq_model *m = nullptr;
    if (jq_qwen3_load_gguf(model_path, n_ctx, &m)) return -2;
    *out_vocab = m->cfg.vocab;
    *out_handle = m;
    return 0;
}

int32_t joshua_npu_forward(void *handle, const uint32_t *tokens, uint32_t n_tokens, uint32_t pos, float *out_logits) {
    if (!handle || !tokens || !out_logits || n_tokens == 0) return -1;
    jq_model *m = (jq_model *)handle;
    // the handle may arrive on another thread than the one that made it; the device is per thread
    if (hipSetDevice(g_device) != hipSuccess) return -5;
    {
        std::lock_guard<std::mutex> lock(m->mu);
        if (pos != m->n_past) return -3;
        if ((uint64_t)pos + n_tokens > m->cfg.n_ctx) return -4;
    }
    return jq_qwen3_forward(m, tokens, n_tokens, pos, out_logits, 0, nullptr) ? -5 : 0;
}

int32_t joshua_npu_reset(void *handle) {
    if (!handle) return -1;
    return jq_qwen3_reset((jq_model *)handle) ? -5 : 0;
}

void joshua_npu_free(void *handle) {
    if (!handle) return;
    (void)hipSetDevice(g_device);
    jq_qwen3_free((jq_model *)handle);
}

}  // extern "C"
