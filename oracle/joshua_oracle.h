/* CPU oracle for the quantized-matmul hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, in plain C, what
 * the reference (rexlunae/joshua, a Rust crate) computes on its x86_64 path so
 * that the HIP kernels can be checked against it.  Only tests/, the smoke
 * check and the benchmark's CPU-baseline leg may load it.
 *
 * Two builds of the same arithmetic live here:
 *   joshua_oracle.c       scalar C; every f32 operation the reference's AVX2
 *                         kernels perform is spelled out with fmaf()/explicit
 *                         rounding, in the reference's lane order, so results
 *                         are bit-identical to the intrinsics build.
 *   joshua_oracle_avx2.c  the same kernels in AVX2/FMA intrinsics with the
 *                         reference's row-chunk thread schedule; this is the
 *                         timed CPU baseline.
 *
 * Pin status of each function (what independent evidence fixes it):
 *   orc_dequantize IQ2_XXS   pinned: llama.cpp golden vectors held by the
 *                            reference (tests/golden/iq2xxs_*.{bin,txt}),
 *                            format bound, table checksum.
 *   orc_dequantize MXFP4     pinned: closed forms (powers of two, E2M1 table,
 *                            split-half nibble order, e=0 / e=0xFF cases).
 *   orc_dequantize Q8_0/Q2_K/Q4_K  pinned: an independent numpy decode written
 *                            from the element-index maps, exhaustive sweeps of
 *                            the 6-bit scale packing and every nibble value.
 *   orc_dequantize Q6_K      pinned on layout by an independent numpy decode
 *                            written from the ggml block definition; the
 *                            reference decodes Q6_K through a third-party
 *                            crate (candle-core ^0.11, k_quants::BlockQ6K::
 *                            to_float) whose source is not available, so the
 *                            ulp-level operation order ((d*sc)*q) is
 *                            PARITY UNPINNED.
 *   orc_decode_raw_to_f32 F16, Q8_K  pinned: numpy's own float16 conversion and d * q written in numpy
 *                             (tests/test_decode_raw.py); Q8_1: parity unpinned (candle-core 0.11's
 *                             BlockQ8_1::to_float is not in the tree; ggml's published layout is used)
 *   orc_dequantize Q4_0/Q4_1/Q5_0/Q5_1/Q3_K/Q5_K  pinned on layout by an
 *                            independent numpy decode written from the block
 *                            definitions and by exhaustive sweeps of every
 *                            field; the values do not depend on the operation
 *                            order (every product is exact in f32, one rounding
 *                            at most per weight), so nothing is left open at
 *                            ulp level.  The reference decodes them through
 *                            candle-core ^0.11 k_quants (not in the container);
 *                            the layouts come from the vendored Metal source.
 *   orc_matmul_t (all)       pinned: equals a float64 GEMM over the decoded
 *                            weights within the reference's own tolerances,
 *                            assign semantics, shape rejection, scalar build
 *                            == AVX2 build bit for bit, thread count
 *                            independence bit for bit.
 */
#ifndef JOSHUA_ORACLE_H
#define JOSHUA_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Raw GGUF tensor-type ids (reference: src/gguf_ext.rs:483-512,
 * src/iq2xxs.rs:23, src/mxfp4.rs:39). */
enum {
    ORC_TYPE_Q8_0 = 8,
    ORC_TYPE_Q2_K = 10,
    ORC_TYPE_Q4_K = 12,
    ORC_TYPE_Q6_K = 14,
    ORC_TYPE_IQ2_XXS = 16,
    ORC_TYPE_MXFP4 = 39,
    /* served by the reference through candle's to_float plus the 8-lane dot
     * (src/quant_matmul.rs:228-248); sizes src/gguf_ext.rs:487-500 */
    ORC_TYPE_Q4_0 = 2,
    ORC_TYPE_Q4_1 = 3,
    ORC_TYPE_Q5_0 = 6,
    ORC_TYPE_Q5_1 = 7,
    ORC_TYPE_Q3_K = 11,
    ORC_TYPE_Q5_K = 13
};

/* Elements and bytes per block of `type`; returns 0, or -1 for an unknown id. */
int orc_block_geometry(uint32_t type, size_t *elems, size_t *bytes);

/* Canonical decode ("to_float") of `nblocks` blocks into out[nblocks*elems]. */
int orc_dequantize(uint32_t type, const void *blocks, size_t nblocks, float *out);
/* 0: decoded; 2: the reference answers None for this type; 1: error (reference: src/quant_matmul.rs:36-103) */
int orc_decode_raw_to_f32(uint32_t dtype, const void *bytes, size_t nbytes, size_t elems, float *out);

/* dst[m,n] = lhs[m,k] . W[n,k]^T in the reference's x86_64 operation order.
 * `lhs_len`/`dst_len` are element counts, `nbytes` the byte length of
 * `blocks`; shape mismatches return nonzero and leave dst untouched
 * (reference: src/quant_matmul.rs:133-165). */
int orc_matmul_t(uint32_t type, size_t m, size_t k, size_t n,
                 const float *lhs, size_t lhs_len,
                 const void *blocks, size_t nbytes,
                 float *dst, size_t dst_len);

/* Same arithmetic in AVX2/FMA intrinsics, rows spread over `threads` workers
 * with the reference's chunking (src/simd.rs:128-145).  threads <= 0 means
 * one worker per online CPU.  Bit-identical to orc_matmul_t. */
int orc_matmul_t_avx2(uint32_t type, size_t m, size_t k, size_t n,
                      const float *lhs, size_t lhs_len,
                      const void *blocks, size_t nbytes,
                      float *dst, size_t dst_len, int threads);

/* The reference's portable IQ2_XXS row worker (per-block sequential sums
 * added into a zero-filled dst; src/iq2xxs.rs:241-268). */
int orc_iq2xxs_matmul_scalar(size_t m, size_t k, size_t n,
                             const float *lhs, size_t lhs_len,
                             const void *blocks, size_t nbytes,
                             float *dst, size_t dst_len);

/* 1 when the AVX2 build is usable on this CPU. */
int orc_have_avx2(void);
/* Worker count the AVX2 build uses for threads <= 0. */
int orc_default_threads(void);

/* Message for the last nonzero return on this thread. */
const char *orc_last_error(void);

#ifdef __cplusplus
}
#endif
#endif
