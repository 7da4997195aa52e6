/* Scalar CPU oracle: see joshua_oracle.h for what this is and how it is pinned.
 * Build with -ffp-contract=off: every fused multiply-add below is explicit. */
#include "joshua_oracle.h"
#include "iq2xxs_grid_codes.h"

#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

static __thread char g_err[256];

const char *orc_last_error(void) { return g_err; }

int orc_fail(const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof g_err, fmt, ap);
    va_end(ap);
    return 1;
}

/* IEEE binary16 -> binary32, exact (the `half` crate's f16::to_f32). */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static inline uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }
static inline uint32_t rd32(const uint8_t *p) {
    return (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}

int orc_block_geometry(uint32_t type, size_t *elems, size_t *bytes) {
    size_t e, b;
    switch (type) { /* reference: src/gguf_ext.rs:483-512 */
    case ORC_TYPE_Q8_0: e = 32; b = 34; break;
    case ORC_TYPE_Q2_K: e = 256; b = 84; break;
    case ORC_TYPE_Q4_K: e = 256; b = 144; break;
    case ORC_TYPE_Q6_K: e = 256; b = 210; break;
    case ORC_TYPE_IQ2_XXS: e = 256; b = 66; break;
    case ORC_TYPE_MXFP4: e = 32; b = 17; break;
    case ORC_TYPE_Q4_0: e = 32; b = 18; break;
    case ORC_TYPE_Q4_1: e = 32; b = 20; break;
    case ORC_TYPE_Q5_0: e = 32; b = 22; break;
    case ORC_TYPE_Q5_1: e = 32; b = 24; break;
    case ORC_TYPE_Q3_K: e = 256; b = 110; break;
    case ORC_TYPE_Q5_K: e = 256; b = 176; break;
    default: return -1;
    }
    if (elems) *elems = e;
    if (bytes) *bytes = b;
    return 0;
}

/* Q4_K 6-bit scale/min pair j of the 12 packed bytes
 * (reference: src/kquant_dot.rs:108-118). */
void orc_q4k_scale_min(const uint8_t *s, int j, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = s[j] & 63;
        *mn = s[j + 4] & 63;
    } else {
        *sc = (uint8_t)((s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4));
        *mn = (uint8_t)((s[j + 4] >> 4) | ((s[j] >> 6) << 4));
    }
}

/* IQ2_XXS codebook entry `code` expanded to its 8 values. */
void orc_iq2xxs_grid(int code, uint8_t out[8]) {
    unsigned c = ORC_IQ2XXS_GRID_TRITS[code];
    for (int j = 0; j < 8; j++) {
        unsigned t = c % 3;
        c /= 3;
        out[j] = (uint8_t)(8 + 17 * t + (t >> 1));
    }
}

/* Sign byte for 7-bit index i: bit 7 makes the popcount even
 * (reference table: src/iq2xxs.rs:441-449). */
uint8_t orc_iq2xxs_signs(unsigned i) {
    return (uint8_t)(i | ((unsigned)(__builtin_popcount(i) & 1) << 7));
}

/* MXFP4 shared exponent (reference: src/mxfp4.rs:67-75); returns 0 and sets
 * *ok = 0 for the reserved 0xFF code. */
float orc_e8m0(uint8_t e, int *ok) {
    uint32_t bits;
    *ok = 1;
    if (e == 0) {
        bits = 0x00400000u;
    } else if (e == 0xFF) {
        *ok = 0;
        bits = 0;
    } else {
        bits = (uint32_t)e << 23;
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

static const float E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                               -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* ---- canonical decode ("to_float") ------------------------------------- */

/* y = q * d (candle BlockQ8_0::to_float; the fused kernel computes the same
 * product, reference: src/kquant_dot.rs:287-302). */
static void deq_q8_0(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b));
    for (int j = 0; j < 32; j++) y[j] = (float)(int8_t)b[2 + j] * d;
}

/* Two rounded operations per element: dl*q - ml
 * (element map, reference: src/kquant_dot.rs:26-29,349-385). */
static void deq_q2_k(const uint8_t *b, float *y) {
    const uint8_t *scales = b, *qs = b + 16;
    float d = orc_f16_to_f32(rd16(b + 80));
    float dmin = orc_f16_to_f32(rd16(b + 82));
    for (int e = 0; e < 256; e++) {
        int sg = e / 128, r = e % 128;
        uint8_t byte = qs[32 * sg + r % 32];
        int q = (byte >> (2 * (r / 32))) & 3;
        uint8_t s = scales[e / 16];
        float dl = d * (float)(s & 0xF);
        float ml = dmin * (float)(s >> 4);
        y[e] = dl * (float)q - ml;
    }
}

/* (element map, reference: src/kquant_dot.rs:30-33,430-465). */
static void deq_q4_k(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b));
    float dmin = orc_f16_to_f32(rd16(b + 2));
    const uint8_t *scales = b + 4, *qs = b + 16;
    for (int e = 0; e < 256; e++) {
        uint8_t sc, mn;
        orc_q4k_scale_min(scales, e / 32, &sc, &mn);
        uint8_t byte = qs[32 * (e / 64) + e % 32];
        int q = ((e / 32) % 2 == 0) ? (byte & 0xF) : (byte >> 4);
        float d1 = d * (float)sc;
        float m1 = dmin * (float)mn;
        y[e] = d1 * (float)q - m1;
    }
}

/* ggml block_q6_K {ql[128], qh[64], scales[16] i8, d f16}
 * (reference: vendor/candle-metal-kernels/src/metal_src/quantized.metal:
 * 198-203,6673-6694).  Operation order (d*sc)*q is the third-party
 * to_float's and is unpinned at ulp level. */
static void deq_q6_k(const uint8_t *b, float *y) {
    const uint8_t *ql = b, *qh = b + 128;
    const int8_t *sc = (const int8_t *)(b + 192);
    float d = orc_f16_to_f32(rd16(b + 208));
    for (int e = 0; e < 256; e++) {
        int h = e / 128, r = e % 128, l = r % 32, t = r / 32;
        uint8_t lo = ql[64 * h + l + 32 * (t & 1)];
        int nib = (t < 2) ? (lo & 0xF) : (lo >> 4);
        int hi2 = (qh[32 * h + l] >> (2 * t)) & 3;
        int q = (nib | (hi2 << 4)) - 32;
        y[e] = d * (float)sc[e / 16] * (float)q;
    }
}

/* The formats below have no kernel in the reference: candle's to_float (third party, not in the
 * container) decodes them and dot_row_avx2 multiplies (src/quant_matmul.rs:228-248).  Layouts and
 * element maps are restated from the vendored Metal source, the one statement of them under
 * /root/reference: vendor/candle-metal-kernels/src/metal_src/quantized.metal:21-61 (structs of the
 * 32-element formats), :151-156 and :176-189 (Q3_K, Q5_K), :6482-6567 and :6597-6670 (element maps).
 * Every product is exact in f32 and each weight is rounded at most once, so the values do not depend
 * on the order of the operations; pinned by tests/np_decode.py on arbitrary bytes and by exhaustive
 * field sweeps. */
static void deq_q4_0(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b));
    for (int j = 0; j < 16; j++) {
        y[j] = (float)((b[2 + j] & 0xF) - 8) * d;
        y[j + 16] = (float)((b[2 + j] >> 4) - 8) * d;
    }
}

static void deq_q4_1(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b)), m = orc_f16_to_f32(rd16(b + 2));
    for (int j = 0; j < 16; j++) {
        y[j] = (float)(b[4 + j] & 0xF) * d + m;
        y[j + 16] = (float)(b[4 + j] >> 4) * d + m;
    }
}

static void deq_q5_0(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b));
    uint32_t qh = rd32(b + 2);
    for (int j = 0; j < 16; j++) {
        int lo = (b[6 + j] & 0xF) | (int)(((qh >> j) & 1u) << 4);
        int hi = (b[6 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
        y[j] = (float)(lo - 16) * d;
        y[j + 16] = (float)(hi - 16) * d;
    }
}

static void deq_q5_1(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b)), m = orc_f16_to_f32(rd16(b + 2));
    uint32_t qh = rd32(b + 4);
    for (int j = 0; j < 16; j++) {
        int lo = (b[8 + j] & 0xF) | (int)(((qh >> j) & 1u) << 4);
        int hi = (b[8 + j] >> 4) | (int)(((qh >> (j + 16)) & 1u) << 4);
        y[j] = (float)lo * d + m;
        y[j + 16] = (float)hi * d + m;
    }
}

/* hmask[32] | qs[64] | scales[12] | d.  Element e = 128 h + 32 t + l: two low bits from field t of
 * qs[32 h + l], third bit = bit 4 h + t of hmask[l] (set: nothing subtracted, clear: 4); sixteen 6-bit
 * scales, one per 16 elements. */
static void deq_q3_k(const uint8_t *b, float *y) {
    const uint8_t *hm = b, *qs = b + 32, *sc = b + 96;
    float d = orc_f16_to_f32(rd16(b + 108));
    for (int e = 0; e < 256; e++) {
        int h = e / 128, t = (e % 128) / 32, l = e % 32, is = e / 16;
        int low4 = is < 8 ? (sc[is] & 0xF) : (sc[is - 8] >> 4);
        int high2 = (sc[8 + is % 4] >> (2 * (is / 4))) & 3;
        int scale = (low4 | (high2 << 4)) - 32;
        int q = ((qs[32 * h + l] >> (2 * t)) & 3) - (((hm[l] >> (4 * h + t)) & 1) ? 0 : 4);
        y[e] = (d * (float)scale) * (float)q;
    }
}

/* d | dmin | scales[12] | qh[32] | qs[128].  Sub-block j (32 elements): nibble (j & 1) of
 * qs[32 (j / 2) + l], fifth bit = bit j of qh[l]; scales and mins packed as in Q4_K. */
static void deq_q5_k(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b)), dmin = orc_f16_to_f32(rd16(b + 2));
    const uint8_t *qh = b + 16, *qs = b + 48;
    for (int j = 0; j < 8; j++) {
        uint8_t sc, mn;
        orc_q4k_scale_min(b + 4, j, &sc, &mn);
        float d1 = d * (float)sc, m1 = dmin * (float)mn;
        for (int l = 0; l < 32; l++) {
            int nib = (j & 1) ? (qs[32 * (j / 2) + l] >> 4) : (qs[32 * (j / 2) + l] & 0xF);
            int q = nib | (((qh[l] >> j) & 1) << 4);
            y[32 * j + l] = d1 * (float)q - m1;
        }
    }
}

/* (reference: src/iq2xxs.rs:44-71). */
static void deq_iq2_xxs(const uint8_t *b, float *y) {
    float d = orc_f16_to_f32(rd16(b));
    const uint8_t *qs = b + 2;
    for (int ib32 = 0; ib32 < 8; ib32++) {
        uint32_t lo = rd32(qs + 8 * ib32);
        uint32_t hi = rd32(qs + 8 * ib32 + 4);
        float db = d * (0.5f + (float)(hi >> 28)) * 0.25f;
        for (int l = 0; l < 4; l++) {
            uint8_t grid[8];
            orc_iq2xxs_grid((lo >> (8 * l)) & 0xFF, grid);
            uint8_t signs = orc_iq2xxs_signs((hi >> (7 * l)) & 127);
            for (int j = 0; j < 8; j++) {
                float s = (signs & (1u << j)) ? -1.0f : 1.0f;
                y[ib32 * 32 + l * 8 + j] = db * (float)grid[j] * s;
            }
        }
    }
}

/* (reference: src/mxfp4.rs:83-94). */
static void deq_mxfp4(const uint8_t *b, float *y) {
    int ok;
    float d = orc_e8m0(b[0], &ok);
    if (!ok) {
        for (int j = 0; j < 32; j++) y[j] = 0.0f;
        return;
    }
    for (int j = 0; j < 16; j++) {
        y[j] = d * E2M1[b[1 + j] & 0xF];
        y[j + 16] = d * E2M1[b[1 + j] >> 4];
    }
}

typedef void (*deq_fn)(const uint8_t *, float *);

static deq_fn deq_for(uint32_t type) {
    switch (type) {
    case ORC_TYPE_Q8_0: return deq_q8_0;
    case ORC_TYPE_Q2_K: return deq_q2_k;
    case ORC_TYPE_Q4_K: return deq_q4_k;
    case ORC_TYPE_Q6_K: return deq_q6_k;
    case ORC_TYPE_IQ2_XXS: return deq_iq2_xxs;
    case ORC_TYPE_MXFP4: return deq_mxfp4;
    case ORC_TYPE_Q4_0: return deq_q4_0;
    case ORC_TYPE_Q4_1: return deq_q4_1;
    case ORC_TYPE_Q5_0: return deq_q5_0;
    case ORC_TYPE_Q5_1: return deq_q5_1;
    case ORC_TYPE_Q3_K: return deq_q3_k;
    case ORC_TYPE_Q5_K: return deq_q5_k;
    default: return NULL;
    }
}

int orc_dequantize(uint32_t type, const void *blocks, size_t nblocks, float *out) {
    size_t elems, bytes;
    deq_fn f = deq_for(type);
    if (!f || orc_block_geometry(type, &elems, &bytes)) return orc_fail("unknown tensor type %u", type);
    const uint8_t *p = (const uint8_t *)blocks;
    for (size_t i = 0; i < nblocks; i++) f(p + i * bytes, out + i * elems);
    return 0;
}


/* decode_raw_to_f32 (reference: src/quant_matmul.rs:36-103): raw tensor bytes of ggml type `dtype` to f32.
 * Returns 0 with `out` filled, 2 where the reference answers None (F32, and every type without a decoder
 * there: the caller keeps its own reader), 1 with a message on a size mismatch.  F16 is converted per
 * element (:71-80); Q8_K is d * q with an f32 d (4 + 256 + 32 bytes a block); Q8_1 is d * q with an f16 d
 * (2 + 2 + 32 bytes a block) by the published ggml layout -- parity unpinned for Q8_1: the reference hands it
 * to candle-core 0.11's BlockQ8_1::to_float, which is not in the tree. */
int orc_decode_raw_to_f32(uint32_t dtype, const void *bytes, size_t nbytes, size_t elems, float *out) {
    const uint8_t *p = (const uint8_t *)bytes;
    if (dtype == 0) return 2;
    if (dtype == 1) {
        if (nbytes != elems * 2) return orc_fail("dtype F16: %zu bytes for %zu elements", nbytes, elems);
        for (size_t i = 0; i < elems; i++) out[i] = orc_f16_to_f32((uint16_t)(p[2 * i] | (p[2 * i + 1] << 8)));
        return 0;
    }
    if (dtype == 9 || dtype == 15) {
        const size_t blck = dtype == 9 ? 32 : 256, bb = dtype == 9 ? 36 : 292;
        if (elems % blck != 0 || nbytes != elems / blck * bb)
            return orc_fail("dtype %u: %zu bytes for %zu elements (%zu per %zu-block)", dtype, nbytes, elems, bb, blck);
        for (size_t b = 0; b < elems / blck; b++) {
            const uint8_t *blk = p + b * bb;
            float d;
            if (dtype == 9) d = orc_f16_to_f32((uint16_t)(blk[0] | (blk[1] << 8)));
            else memcpy(&d, blk, 4);
            const int8_t *q = (const int8_t *)(blk + 4);
            for (size_t e = 0; e < blck; e++) out[b * blck + e] = d * (float)q[e];
        }
        return 0;
    }
    size_t be, bb;
    if (!deq_for(dtype) || orc_block_geometry(dtype, &be, &bb)) return 2;
    if (elems % be != 0 || nbytes != elems / be * bb)
        return orc_fail("dtype %u: %zu bytes for %zu elements (%zu per %zu-block)", dtype, nbytes, elems, bb, be);
    return orc_dequantize(dtype, bytes, elems / be, out);
}

/* ---- matmul in the reference's x86_64 operation order ------------------ */

/* Shared shape check (reference: src/quant_matmul.rs:133-165,
 * src/iq2xxs.rs:126-153, src/mxfp4.rs:142-172).  Returns blocks per row
 * through *bpr. */
int orc_validate(uint32_t type, size_t m, size_t k, size_t n, size_t lhs_len, size_t nbytes,
                 size_t dst_len, size_t *bpr) {
    size_t elems, bytes;
    if (orc_block_geometry(type, &elems, &bytes)) return orc_fail("unknown tensor type %u", type);
    if (k % elems != 0)
        return orc_fail("quantized matmul: k=%zu is not a multiple of the block size %zu", k, elems);
    size_t per_row = k / elems;
    if (nbytes % bytes != 0 || nbytes / bytes != n * per_row)
        return orc_fail("quantized matmul: rhs holds %zu bytes, expected %zu blocks of %zu", nbytes,
                        n * per_row, bytes);
    if (lhs_len != m * k || dst_len != m * n)
        return orc_fail("quantized matmul: lhs/dst sized %zu/%zu expected %zu/%zu", lhs_len, dst_len,
                        m * k, m * n);
    *bpr = per_row;
    return 0;
}

/* The AVX2 horizontal sum (reference: src/simd.rs:198-206). */
static inline float hsum8(const float a[8]) {
    float s0 = a[0] + a[4], s1 = a[1] + a[5], s2 = a[2] + a[6], s3 = a[3] + a[7];
    return (s0 + s2) + (s1 + s3);
}

/* One output element with the 8-lane accumulate of every AVX2 row kernel:
 * lane c%8 takes column c, in column order. */
static float dot8(const float *x, const float *w, size_t k) {
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (size_t c = 0; c < k; c++) acc[c & 7] = fmaf(x[c], w[c], acc[c & 7]);
    return hsum8(acc);
}

/* Row decode as the fused kernels do it in registers. */

/* w = q*d, one rounding (reference: src/kquant_dot.rs:287-302). */
static void fused_w_q8_0(const uint8_t *b, float *w) {
    float d = orc_f16_to_f32(rd16(b));
    for (int j = 0; j < 32; j++) w[j] = (float)(int8_t)b[2 + j] * d;
}

/* w = fmsub(q, d*(s&15), dmin*(s>>4)) (reference: src/kquant_dot.rs:345-385). */
static void fused_w_q2_k(const uint8_t *b, float *w) {
    const uint8_t *scales = b, *qs = b + 16;
    float d = orc_f16_to_f32(rd16(b + 80));
    float dmin = orc_f16_to_f32(rd16(b + 82));
    for (int sg = 0; sg < 2; sg++) {
        for (int j = 0; j < 8; j++) {
            uint8_t s = scales[sg * 8 + j];
            float d1 = d * (float)(s & 0xF);
            float m1 = dmin * (float)(s >> 4);
            int shift = 2 * (j / 2);
            const uint8_t *win = qs + sg * 32 + ((j % 2) ? 16 : 0);
            for (int i = 0; i < 16; i++) {
                float q = (float)((win[i] >> shift) & 3);
                w[sg * 128 + 16 * j + i] = fmaf(q, d1, -m1);
            }
        }
    }
}

/* w = fmsub(q, d*sc, dmin*m) (reference: src/kquant_dot.rs:426-466). */
static void fused_w_q4_k(const uint8_t *b, float *w) {
    float d = orc_f16_to_f32(rd16(b));
    float dmin = orc_f16_to_f32(rd16(b + 2));
    const uint8_t *scales = b + 4, *qs = b + 16;
    for (int c = 0; c < 4; c++) {
        for (int r = 0; r < 2; r++) {
            uint8_t sc, mn;
            orc_q4k_scale_min(scales, 2 * c + r, &sc, &mn);
            float d1 = d * (float)sc;
            float m1 = dmin * (float)mn;
            for (int i = 0; i < 32; i++) {
                uint8_t byte = qs[c * 32 + i];
                float q = (float)(r == 0 ? (byte & 0xF) : (byte >> 4));
                w[64 * c + 32 * r + i] = fmaf(q, d1, -m1);
            }
        }
    }
}

/* v = (grid*sign)*db (reference: src/iq2xxs.rs:349-380). */
static void fused_w_iq2_xxs(const uint8_t *b, float *w) {
    float d = orc_f16_to_f32(rd16(b));
    const uint8_t *qs = b + 2;
    for (int ib32 = 0; ib32 < 8; ib32++) {
        uint32_t lo = rd32(qs + 8 * ib32);
        uint32_t hi = rd32(qs + 8 * ib32 + 4);
        float db = d * (0.5f + (float)(hi >> 28)) * 0.25f;
        for (int l = 0; l < 4; l++) {
            uint8_t grid[8];
            orc_iq2xxs_grid((lo >> (8 * l)) & 0xFF, grid);
            uint8_t signs = orc_iq2xxs_signs((hi >> (7 * l)) & 0x7F);
            for (int j = 0; j < 8; j++) {
                float s = (signs & (1u << j)) ? -1.0f : 1.0f;
                w[ib32 * 32 + l * 8 + j] = ((float)grid[j] * s) * db;
            }
        }
    }
}

int orc_matmul_t(uint32_t type, size_t m, size_t k, size_t n, const float *lhs, size_t lhs_len,
                 const void *blocks, size_t nbytes, float *dst, size_t dst_len) {
    size_t bpr;
    if (orc_validate(type, m, k, n, lhs_len, nbytes, dst_len, &bpr)) return 1;
    if (m == 0 || n == 0) return 0; /* reference: src/quant_matmul.rs:176-178 */
    size_t elems, bytes;
    orc_block_geometry(type, &elems, &bytes);
    const uint8_t *base = (const uint8_t *)blocks;

    if (type == ORC_TYPE_MXFP4) {
        /* Scalar only in the reference: per block a sequential sum with two
         * roundings per term, added into a zero-filled dst
         * (reference: src/mxfp4.rs:185-235). */
        memset(dst, 0, dst_len * sizeof(float));
        float w[32];
        for (size_t row = 0; row < n; row++) {
            for (size_t b = 0; b < bpr; b++) {
                deq_mxfp4(base + (row * bpr + b) * 17, w);
                for (size_t i = 0; i < m; i++) {
                    const float *a = lhs + i * k + b * 32;
                    float acc = 0.0f;
                    for (int j = 0; j < 32; j++) acc += a[j] * w[j];
                    dst[i * n + row] += acc;
                }
            }
        }
        return 0;
    }

    void (*rowdec)(const uint8_t *, float *);
    switch (type) {
    case ORC_TYPE_Q8_0: rowdec = fused_w_q8_0; break;
    case ORC_TYPE_Q2_K: rowdec = fused_w_q2_k; break;
    case ORC_TYPE_Q4_K: rowdec = fused_w_q4_k; break;
    case ORC_TYPE_IQ2_XXS: rowdec = fused_w_iq2_xxs; break;
    /* No fused kernel: to_float into a k-float scratch, then the 8-lane dot
     * (reference: src/quant_matmul.rs:228-248,292-325). */
    case ORC_TYPE_Q6_K: rowdec = deq_q6_k; break;
    case ORC_TYPE_Q4_0: rowdec = deq_q4_0; break;
    case ORC_TYPE_Q4_1: rowdec = deq_q4_1; break;
    case ORC_TYPE_Q5_0: rowdec = deq_q5_0; break;
    case ORC_TYPE_Q5_1: rowdec = deq_q5_1; break;
    case ORC_TYPE_Q3_K: rowdec = deq_q3_k; break;
    case ORC_TYPE_Q5_K: rowdec = deq_q5_k; break;
    default: return orc_fail("unknown tensor type %u", type);
    }
    float *w = (float *)malloc(k * sizeof(float));
    if (!w) return orc_fail("out of memory");
    for (size_t row = 0; row < n; row++) {
        for (size_t b = 0; b < bpr; b++) rowdec(base + (row * bpr + b) * bytes, w + b * elems);
        for (size_t i = 0; i < m; i++) dst[i * n + row] = dot8(lhs + i * k, w, k);
    }
    free(w);
    return 0;
}

int orc_iq2xxs_matmul_scalar(size_t m, size_t k, size_t n, const float *lhs, size_t lhs_len,
                             const void *blocks, size_t nbytes, float *dst, size_t dst_len) {
    size_t bpr;
    if (orc_validate(ORC_TYPE_IQ2_XXS, m, k, n, lhs_len, nbytes, dst_len, &bpr)) return 1;
    if (m == 0 || n == 0) return 0;
    memset(dst, 0, dst_len * sizeof(float));
    const uint8_t *base = (const uint8_t *)blocks;
    float w[256];
    for (size_t row = 0; row < n; row++) {
        for (size_t b = 0; b < bpr; b++) {
            deq_iq2_xxs(base + (row * bpr + b) * 66, w);
            for (size_t i = 0; i < m; i++) {
                const float *a = lhs + i * k + b * 256;
                float acc = 0.0f;
                for (int j = 0; j < 256; j++) acc += a[j] * w[j];
                dst[i * n + row] += acc;
            }
        }
    }
    return 0;
}
