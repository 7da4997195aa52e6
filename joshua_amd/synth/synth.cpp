// Synthetic-input tooling for tests and benchmarks: a counter-based seeded
// normal/uniform generator and host-side block quantizers that turn f32
// matrices into GGUF blocks (Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4).
//
// The reference has no quantizers on this path (it quantizes only in tests,
// through the third-party candle-core crate), so the block bytes produced here
// are this build's own: round-to-nearest encoders in the style of ggml's
// reference quantizers.  Matmul parity is always defined on identical block
// bytes, whatever produced them.  Host only; nothing here touches the GPU.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

#include "../csrc/iq2xxs_grid_codes.h"

namespace {

inline uint64_t splitmix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// Two standard normals for pair index p of stream `seed` (Box-Muller).
inline void normal_pair(uint64_t seed, uint64_t p, float *z0, float *z1) {
    uint64_t h = splitmix64(splitmix64(seed) ^ (p * 0xD1342543DE82EF95ull + 0x2545F4914F6CDD1Dull));
    uint32_t a = (uint32_t)(h >> 32), b = (uint32_t)h;
    float u1 = ((float)(a >> 8) + 1.0f) * (1.0f / 16777216.0f);  // (0, 1]
    float u2 = (float)(b >> 8) * (1.0f / 16777216.0f);           // [0, 1)
    float r = std::sqrt(-2.0f * std::log(u1));
    float t = 6.28318530717958647692f * u2;
    *z0 = r * std::cos(t);
    *z1 = r * std::sin(t);
}

inline float normal_at(uint64_t seed, uint64_t i) {
    float z0, z1;
    normal_pair(seed, i >> 1, &z0, &z1);
    return (i & 1) ? z1 : z0;
}

template <class F>
void parallel_ranges(size_t n, size_t grain, int threads, F f) {
    if (threads <= 0) threads = (int)std::max(1u, std::thread::hardware_concurrency());
    size_t units = (n + grain - 1) / grain;
    size_t nt = std::min<size_t>((size_t)threads, std::max<size_t>(units, 1));
    if (nt <= 1) {
        f((size_t)0, n);
        return;
    }
    std::vector<std::thread> pool;
    size_t per = (units + nt - 1) / nt;
    for (size_t t = 0; t < nt; t++) {
        size_t b = std::min(n, t * per * grain), e = std::min(n, (t + 1) * per * grain);
        if (b < e) pool.emplace_back([=] { f(b, e); });
    }
    for (auto &th : pool) th.join();
}

uint16_t f32_to_f16(float f) {  // round to nearest even
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    int32_t exp = (int32_t)((x >> 23) & 0xFF) - 127 + 15;
    uint32_t man = x & 0x7FFFFFu;
    if (((x >> 23) & 0xFF) == 0xFF) return (uint16_t)(sign | 0x7C00u | (man ? 0x200u : 0));
    if (exp >= 31) return (uint16_t)(sign | 0x7C00u);
    if (exp <= 0) {
        if (exp < -10) return (uint16_t)sign;
        man |= 0x800000u;
        int shift = 14 - exp;
        uint32_t half = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1), mid = 1u << (shift - 1);
        if (rem > mid || (rem == mid && (half & 1))) half++;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)exp << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;
    return (uint16_t)(sign | half);
}

float f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1F, man = h & 0x3FF, bits;
    if (exp == 0) {
        if (!man) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FF) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
    else bits = sign | ((exp + 112) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline int nearest_int(float v) { return (int)std::lrintf(v); }
inline void put16(uint8_t *p, uint16_t v) { p[0] = (uint8_t)v; p[1] = (uint8_t)(v >> 8); }

// ---- Q8_0: d = amax/127, q = round(x/d) -------------------------------------
void quant_q8_0(const float *x, uint8_t *out) {
    float amax = 0;
    for (int j = 0; j < 32; j++) amax = std::max(amax, std::fabs(x[j]));
    float d = amax / 127.0f, id = d ? 1.0f / d : 0.0f;
    put16(out, f32_to_f16(d));
    for (int j = 0; j < 32; j++) out[2 + j] = (uint8_t)(int8_t)nearest_int(x[j] * id);
}

// Iterated scale/min fit of x ~ scale*L - min, L in [0, nmax].
float fit_scale_min(int n, int nmax, const float *x, uint8_t *L, float *the_min, int ntry) {
    float mn = x[0], mx = x[0];
    for (int i = 1; i < n; i++) { mn = std::min(mn, x[i]); mx = std::max(mx, x[i]); }
    if (mx == mn) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = 0;
        return 0;
    }
    if (mn > 0) mn = 0;
    float iscale = nmax / (mx - mn), scale = 1 / iscale;
    for (int it = 0; it < ntry; it++) {
        float sumlx = 0;
        int suml2 = 0;
        bool changed = false;
        for (int i = 0; i < n; i++) {
            int l = std::max(0, std::min(nmax, nearest_int(iscale * (x[i] - mn))));
            if (l != L[i]) { L[i] = (uint8_t)l; changed = true; }
            sumlx += (x[i] - mn) * l;
            suml2 += l * l;
        }
        scale = sumlx / suml2;
        float sum = 0;
        for (int i = 0; i < n; i++) sum += x[i] - scale * L[i];
        mn = 0.5f * mn + 0.5f * sum / n;
        if (mn > 0) mn = 0;
        iscale = 1 / scale;
        if (!changed) break;
    }
    *the_min = -mn;
    return scale;
}

void quant_q4_k(const float *x, uint8_t *out) {
    uint8_t L[256] = {0};
    float scales[8], mins[8], max_scale = 0, max_min = 0;
    for (int j = 0; j < 8; j++) {
        scales[j] = fit_scale_min(32, 15, x + 32 * j, L + 32 * j, &mins[j], 5);
        max_scale = std::max(max_scale, scales[j]);
        max_min = std::max(max_min, mins[j]);
    }
    float inv_scale = max_scale > 0 ? 63.0f / max_scale : 0, inv_min = max_min > 0 ? 63.0f / max_min : 0;
    uint8_t *sc = out + 4;
    std::memset(sc, 0, 12);
    for (int j = 0; j < 8; j++) {
        uint8_t ls = (uint8_t)std::min(63, nearest_int(inv_scale * scales[j]));
        uint8_t lm = (uint8_t)std::min(63, nearest_int(inv_min * mins[j]));
        if (j < 4) {
            sc[j] = ls;
            sc[j + 4] = lm;
        } else {
            sc[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
            sc[j - 4] |= (uint8_t)((ls >> 4) << 6);
            sc[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    uint16_t dh = f32_to_f16(max_scale / 63.0f), mh = f32_to_f16(max_min / 63.0f);
    put16(out, dh);
    put16(out + 2, mh);
    float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    for (int j = 0; j < 8; j++) {
        uint8_t s, m;
        if (j < 4) { s = sc[j] & 63; m = sc[j + 4] & 63; }
        else { s = (uint8_t)((sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)); m = (uint8_t)((sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)); }
        float d1 = d * s;
        if (d1 == 0) continue;
        float dm = dmin * m;
        for (int i = 0; i < 32; i++)
            L[32 * j + i] = (uint8_t)std::max(0, std::min(15, nearest_int((x[32 * j + i] + dm) / d1)));
    }
    uint8_t *q = out + 16;
    for (int c = 0; c < 4; c++)
        for (int l = 0; l < 32; l++) q[32 * c + l] = (uint8_t)(L[64 * c + l] | (L[64 * c + 32 + l] << 4));
}

void quant_q2_k(const float *x, uint8_t *out) {
    uint8_t L[256] = {0};
    float scales[16], mins[16], max_scale = 0, max_min = 0;
    for (int j = 0; j < 16; j++) {
        scales[j] = fit_scale_min(16, 3, x + 16 * j, L + 16 * j, &mins[j], 5);
        max_scale = std::max(max_scale, scales[j]);
        max_min = std::max(max_min, mins[j]);
    }
    uint8_t *sc = out;
    uint16_t dh = 0, mh = 0;
    std::memset(sc, 0, 16);
    if (max_scale > 0) {
        float is = 15.0f / max_scale;
        for (int j = 0; j < 16; j++) sc[j] = (uint8_t)std::min(15, nearest_int(is * scales[j]));
        dh = f32_to_f16(max_scale / 15.0f);
    }
    if (max_min > 0) {
        float is = 15.0f / max_min;
        for (int j = 0; j < 16; j++) sc[j] |= (uint8_t)(std::min(15, nearest_int(is * mins[j])) << 4);
        mh = f32_to_f16(max_min / 15.0f);
    }
    put16(out + 80, dh);
    put16(out + 82, mh);
    float d = f16_to_f32(dh), dmin = f16_to_f32(mh);
    for (int j = 0; j < 16; j++) {
        float d1 = d * (sc[j] & 0xF);
        if (d1 == 0) continue;
        float dm = dmin * (sc[j] >> 4);
        for (int i = 0; i < 16; i++)
            L[16 * j + i] = (uint8_t)std::max(0, std::min(3, nearest_int((x[16 * j + i] + dm) / d1)));
    }
    uint8_t *q = out + 16;
    for (int sg = 0; sg < 2; sg++)
        for (int l = 0; l < 32; l++)
            q[32 * sg + l] = (uint8_t)(L[128 * sg + l] | (L[128 * sg + l + 32] << 2) |
                                       (L[128 * sg + l + 64] << 4) | (L[128 * sg + l + 96] << 6));
}

// Symmetric fit x ~ scale*(L - nmax), L in [0, 2*nmax), weighted by x^2.
float fit_symmetric(int n, int nmax, const float *x, int8_t *L) {
    float mx = 0, amax = 0;
    for (int i = 0; i < n; i++) {
        float ax = std::fabs(x[i]);
        if (ax > amax) { amax = ax; mx = x[i]; }
    }
    if (amax < 1e-30f) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0;
    }
    float best = 0, scale = 0;
    // Try the plain -nmax/max scaling first, then 18 perturbed ones; a
    // perturbation wins only when it strictly lowers the weighted error.
    for (int it = 0; it < 19; it++) {
        int step = it == 0 ? 0 : (it <= 9 ? it - 10 : it - 9);
        float iscale = -(nmax + 0.1f * step) / mx;
        float sumlx = 0, suml2 = 0;
        int8_t cand[32];
        for (int i = 0; i < n; i++) {
            int l = std::max(-nmax, std::min(nmax - 1, nearest_int(iscale * x[i])));
            cand[i] = (int8_t)l;
            float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && (it == 0 || sumlx * sumlx > best * suml2)) {
            scale = sumlx / suml2;
            best = scale * sumlx;
            for (int i = 0; i < n; i++) L[i] = cand[i];
        }
    }
    return scale;
}

void quant_q6_k(const float *x, uint8_t *out) {
    int8_t L[256];
    float scales[16], max_scale = 0, max_abs = 0;
    for (int ib = 0; ib < 16; ib++) {
        scales[ib] = fit_symmetric(16, 32, x + 16 * ib, L + 16 * ib);
        if (std::fabs(scales[ib]) > max_abs) { max_abs = std::fabs(scales[ib]); max_scale = scales[ib]; }
    }
    uint8_t *ql = out, *qh = out + 128;
    int8_t *sc = (int8_t *)(out + 192);
    if (max_abs < 1e-30f) {
        std::memset(out, 0, 210);
        return;
    }
    float iscale = -128.0f / max_scale;
    uint16_t dh = f32_to_f16(1 / iscale);
    put16(out + 208, dh);
    float d = f16_to_f32(dh);
    uint8_t U[256];
    for (int ib = 0; ib < 16; ib++) {
        sc[ib] = (int8_t)std::min(127, nearest_int(iscale * scales[ib]));
        float d1 = d * sc[ib];
        for (int i = 0; i < 16; i++) {
            int l = d1 != 0 ? std::max(-32, std::min(31, nearest_int(x[16 * ib + i] / d1))) : 0;
            U[16 * ib + i] = (uint8_t)(l + 32);
        }
    }
    for (int h = 0; h < 2; h++) {
        const uint8_t *u = U + 128 * h;
        for (int l = 0; l < 32; l++) {
            ql[64 * h + l] = (uint8_t)((u[l] & 0xF) | ((u[l + 64] & 0xF) << 4));
            ql[64 * h + l + 32] = (uint8_t)((u[l + 32] & 0xF) | ((u[l + 96] & 0xF) << 4));
            qh[32 * h + l] = (uint8_t)((u[l] >> 4) | ((u[l + 32] >> 4) << 2) | ((u[l + 64] >> 4) << 4) |
                                       ((u[l + 96] >> 4) << 6));
        }
    }
}

// ---- IQ2_XXS: nearest codebook entry per 8 values -----------------------------
struct GridTable {
    float v[256][8];
    GridTable() {
        for (int i = 0; i < 256; i++) {
            unsigned c = JQ_IQ2XXS_GRID_TRITS[i];
            for (int j = 0; j < 8; j++) {
                unsigned t = c % 3;
                c /= 3;
                v[i][j] = (float)(8 + 17 * t + (t >> 1));
            }
        }
    }
};
const GridTable &grid_table() {
    static GridTable g;
    return g;
}

void quant_iq2_xxs(const float *x, uint8_t *out) {
    const GridTable &G = grid_table();
    float amax = 0;
    for (int i = 0; i < 256; i++) amax = std::max(amax, std::fabs(x[i]));
    // Largest decodable magnitude is d * (0.5 + 15) * 0.25 * 43.
    uint16_t dh = f32_to_f16(amax / (15.5f * 0.25f * 43.0f));
    put16(out, dh);
    float d = f16_to_f32(dh);
    for (int g = 0; g < 8; g++) {
        const float *xg = x + 32 * g;
        float gmax = 0;
        for (int i = 0; i < 32; i++) gmax = std::max(gmax, std::fabs(xg[i]));
        int s4 = 0;
        if (d > 0) s4 = std::max(0, std::min(15, nearest_int(gmax / (43.0f * 0.25f * d) - 0.5f)));
        float db = d * (0.5f + (float)s4) * 0.25f, idb = db > 0 ? 1.0f / db : 0.0f;
        uint32_t lo = 0, hi = (uint32_t)s4 << 28;
        for (int l = 0; l < 4; l++) {
            float t[8];
            unsigned neg = 0;
            int weakest = 0;
            for (int j = 0; j < 8; j++) {
                float v = xg[8 * l + j];
                t[j] = std::fabs(v) * idb;
                if (v < 0) neg |= 1u << j;
                if (t[j] < t[weakest]) weakest = j;
            }
            // Only sign patterns with an even number of minus signs exist.
            if (__builtin_popcount(neg) & 1) neg ^= 1u << weakest;
            int bestc = 0;
            float beste = 1e30f;
            for (int c = 0; c < 256; c++) {
                float e = 0;
                for (int j = 0; j < 8; j++) {
                    float df = G.v[c][j] - t[j];
                    e += df * df;
                }
                if (e < beste) { beste = e; bestc = c; }
            }
            lo |= (uint32_t)bestc << (8 * l);
            hi |= (uint32_t)(neg & 127) << (7 * l);
        }
        std::memcpy(out + 2 + 8 * g, &lo, 4);
        std::memcpy(out + 2 + 8 * g + 4, &hi, 4);
    }
}

// ---- MXFP4: shared power-of-two scale, nearest E2M1 code ------------------------
void quant_mxfp4(const float *x, uint8_t *out) {
    static const float mag[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};
    float amax = 0;
    for (int i = 0; i < 32; i++) amax = std::max(amax, std::fabs(x[i]));
    int e = 127;
    if (amax > 0) {
        int ex;
        std::frexp(amax, &ex);  // amax = f * 2^ex, f in [0.5, 1)
        e = std::max(1, std::min(254, (ex - 1) - 2 + 127));
    }
    out[0] = (uint8_t)e;
    float inv = std::ldexp(1.0f, 127 - e);
    uint8_t code[32];
    for (int i = 0; i < 32; i++) {
        float a = std::fabs(x[i]) * inv;
        int best = 0;
        for (int c = 1; c < 8; c++)
            if (std::fabs(mag[c] - a) < std::fabs(mag[best] - a)) best = c;
        code[i] = (uint8_t)(best | (x[i] < 0 ? 8 : 0));
    }
    for (int j = 0; j < 16; j++) out[1 + j] = (uint8_t)(code[j] | (code[j + 16] << 4));
}

struct Geometry { size_t elems, bytes; void (*fn)(const float *, uint8_t *); };

bool geometry(uint32_t type, Geometry *g) {
    switch (type) {
    case 8: *g = {32, 34, quant_q8_0}; return true;
    case 10: *g = {256, 84, quant_q2_k}; return true;
    case 12: *g = {256, 144, quant_q4_k}; return true;
    case 14: *g = {256, 210, quant_q6_k}; return true;
    case 16: *g = {256, 66, quant_iq2_xxs}; return true;
    case 39: *g = {32, 17, quant_mxfp4}; return true;
    default: return false;
    }
}

}  // namespace

extern "C" {

// out[i] = mean + sigma * z(seed, start + i); the value depends only on
// (seed, start + i), never on the thread count.
int jsyn_fill_normal(uint64_t seed, uint64_t start, size_t n, float mean, float sigma, float *out,
                     int threads) {
    parallel_ranges(n, 4096, threads, [=](size_t b, size_t e) {
        for (size_t i = b; i < e; i++) out[i] = mean + sigma * normal_at(seed, start + i);
    });
    return 0;
}

// out[i] uniform in [0, bound).
int jsyn_fill_uniform_u32(uint64_t seed, uint64_t start, size_t n, uint32_t bound, uint32_t *out) {
    for (size_t i = 0; i < n; i++)
        out[i] = (uint32_t)(((splitmix64(splitmix64(seed) ^ (start + i)) >> 32) * (uint64_t)bound) >> 32);
    return 0;
}

// Bytes needed for n_elems elements of `type`; 0 when the type is unknown or
// n_elems is not a whole number of blocks.
size_t jsyn_quantized_size(uint32_t type, size_t n_elems) {
    Geometry g;
    if (!geometry(type, &g) || n_elems % g.elems) return 0;
    return n_elems / g.elems * g.bytes;
}

int jsyn_quantize(uint32_t type, const float *src, size_t n_elems, void *out, int threads) {
    Geometry g;
    if (!geometry(type, &g) || n_elems % g.elems) return 1;
    uint8_t *o = (uint8_t *)out;
    size_t nblocks = n_elems / g.elems;
    parallel_ranges(nblocks, 64, threads, [=](size_t b, size_t e) {
        for (size_t i = b; i < e; i++) g.fn(src + i * g.elems, o + i * g.bytes);
    });
    return 0;
}

// Quantize mean + sigma*z(seed, start+i) without materialising the f32 matrix.
int jsyn_normal_quantized(uint32_t type, uint64_t seed, uint64_t start, size_t n_elems, float mean,
                          float sigma, void *out, int threads) {
    Geometry g;
    if (!geometry(type, &g) || n_elems % g.elems) return 1;
    uint8_t *o = (uint8_t *)out;
    size_t nblocks = n_elems / g.elems;
    parallel_ranges(nblocks, 64, threads, [=](size_t b, size_t e) {
        float buf[256];
        for (size_t i = b; i < e; i++) {
            for (size_t j = 0; j < g.elems; j++) buf[j] = mean + sigma * normal_at(seed, start + i * g.elems + j);
            g.fn(buf, o + i * g.bytes);
        }
    });
    return 0;
}

}  // extern "C"
