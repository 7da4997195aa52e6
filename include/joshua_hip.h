/* joshua_hip.h — C ABI of libjoshua_hip.so: GGUF quantized matmul on one
 * MI355X (gfx950).
 *
 * The entry points mirror, one to one, the operator contract the reference
 * engine calls on its quantized-weight storage objects
 * (reference: src/mmap_tensor.rs:127-203, trait methods dtype / matmul_t /
 * embedding / dequantize / storage_size_in_bytes, and the free functions
 * src/quant_matmul.rs:110-118 matmul_kquant, src/kquant_dot.rs:126-143
 * try_matmul_fused, src/iq2xxs.rs:103-111 matmul_t, src/mxfp4.rs:120-128
 * matmul_t).  A Rust `QuantizedType` implementation binds them with a plain
 * `extern "C"` block; no C++ or torch types cross this boundary.
 *
 * Conventions
 *   - Every function returns 0 on success and nonzero on failure (the
 *     convention of the reference's plugin ABI, src/npu/mod.rs:48-50).  On
 *     failure nothing has been written to the destination and
 *     jq_last_error() describes the problem (thread local), in the words of
 *     the reference's `bail!` messages where one exists.
 *   - dst[m,n] = lhs[m,k] . W[n,k]^T, all row-major, dst[i*n + j]; dst is
 *     assigned, never accumulated into (reference: src/quant_matmul.rs:105-109,
 *     src/mxfp4.rs:185-189).
 *   - Blocks stay in their native packed GGUF layout in HBM; no f32 copy of a
 *     weight is ever made.
 *   - `stream` is a hipStream_t passed as void*; NULL means the default
 *     stream.  Calls only enqueue work unless they take host pointers.
 *   - A jq_weight is immutable after creation and may be used by several host
 *     threads at once (reference: src/mmap_tensor.rs:86-91).
 */
#ifndef JOSHUA_HIP_H
#define JOSHUA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Raw GGUF tensor type ids (reference: src/gguf_ext.rs:483-512,
 * src/iq2xxs.rs:23, src/mxfp4.rs:39). */
#define JQ_TYPE_Q8_0 8u
#define JQ_TYPE_Q2_K 10u
#define JQ_TYPE_Q4_K 12u
#define JQ_TYPE_Q6_K 14u
#define JQ_TYPE_IQ2_XXS 16u
#define JQ_TYPE_MXFP4 39u
/* Formats the reference serves through the canonical decode plus the 8-lane dot
 * (reference: src/quant_matmul.rs:228-248; sizes src/gguf_ext.rs:487-500). */
#define JQ_TYPE_Q4_0 2u
#define JQ_TYPE_Q4_1 3u
#define JQ_TYPE_Q5_0 6u
#define JQ_TYPE_Q5_1 7u
#define JQ_TYPE_Q3_K 11u
#define JQ_TYPE_Q5_K 13u

typedef struct jq_weight jq_weight;

/* Message for the last failure on the calling thread
 * (replaces candle's Error::Msg strings). */
const char *jq_last_error(void);

/* Name of the kernel that the calling thread's last jq_matmul_t / jq_matmul_t_noalloc /
 * jq_try_matmul_fused call chose ("" before the first one): which kernel serves a shape
 * depends on measured crossover points, and tests pin the choice with this
 * (no counterpart in the reference, which has one kernel per format). */
const char *jq_last_kernel(void);

/* Elements and bytes per block of a type id; nonzero for an unknown id
 * (reference: src/gguf_ext.rs:483-512 type_size_bytes). */
int jq_block_geometry(uint32_t ggml_type, size_t *elems, size_t *bytes);

/* Selects the HIP device for this process and builds the constant tables.
 * Optional: the first upload does it for device 0. */
int jq_init(int device);

/* Copies `nbytes` of packed blocks for an n x k weight (a tensor, or one
 * expert's slice of the mapping) into HBM, once.  `blocks` is a host pointer
 * when src_is_device == 0, else a device pointer.  Fails unless
 * nbytes == n * k / block_elems * block_bytes
 * (reference: src/mmap_tensor.rs:520-565 borrowed_qtensor_raw,
 * src/mmap_tensor.rs:105-123 borrow bounds check). */
int jq_upload(uint32_t ggml_type, const void *blocks, size_t nbytes, size_t n, size_t k,
              int src_is_device, jq_weight **out);

/* A weight that aliases `nbytes` at `byte_offset` inside `parent` without
 * copying: one expert of a stacked [n_expert, n, k] tensor
 * (reference: src/quantized_qwen3_moe.rs:596-631 split_experts,
 * src/mmap_tensor.rs:614-655 borrowed_range).  The parent must outlive it. */
int jq_view(const jq_weight *parent, size_t byte_offset, size_t n, size_t k, jq_weight **out);

void jq_free(jq_weight *w);

/* Accessors (reference: src/mmap_tensor.rs:128-130,175-189). */
uint32_t jq_dtype(const jq_weight *w);
size_t jq_rows(const jq_weight *w);
size_t jq_cols(const jq_weight *w);
size_t jq_storage_size_in_bytes(const jq_weight *w);
const void *jq_device_ptr(const jq_weight *w);

/* THE call: dst[m,n] = lhs[m,k] . W^T.  lhs_len / dst_len are element counts
 * and must equal m*k / m*n; m == 0 or n == 0 succeeds without work
 * (reference: src/mmap_tensor.rs:132-134 matmul_t,
 * src/quant_matmul.rs:133-178 validate + empty case).  With
 * ptrs_are_device == 0 the call stages lhs/dst through HBM and returns after
 * the result has landed in dst.
 * Accuracy: |dst - ref| <= 1e-3 * max(|ref|, 1) against the reference's f32 arithmetic
 * (its own bound, src/kquant_dot.rs:853).  The integer kernels hold the activations in
 * 16-bit fixed point: one scale per 32 elements of a row for Q4_K up to 63 activation rows
 * and for every one-row product, so a row whose groups span many orders of magnitude keeps
 * the bound; the matrix-core GEMM (Q4_K from 64 rows on; every other format from 17 rows
 * on, and from 8 against 8M weights or more) uses one scale per 256 elements, which
 * resolves each super-block to 2^-16 of its largest magnitude (2^-12 of the sum of the
 * terms' magnitudes on such rows; the reference's integer path quantises activations to 8
 * bits per 256, src/quant_matmul.rs:184).  In that GEMM the formats with a scale per 32
 * elements (Q8_0, MXFP4, Q4_0, Q4_1, Q5_0, Q5_1) have the eight blocks of a 256-run put on
 * the run's largest scale at 15 or 16 bits: exact where the scales are equal or a few powers
 * of two apart, else each weight to 2^-15 of the run's largest magnitude or better.  A row
 * holding an inf or a NaN comes out all NaN. */
int jq_matmul_t(const jq_weight *w, size_t m, const float *lhs, size_t lhs_len, float *dst,
                size_t dst_len, int ptrs_are_device, void *stream);

/* The same product over f16 activations into f16 results, elements as IEEE binary16 bit
 * patterns: lhs is widened to f32, multiplied as jq_matmul_t does, and the f32 result is
 * rounded to f16 (nearest even, overflow to infinity) (reference:
 * src/mmap_tensor.rs:136-138, :378-380, :451-453 matmul_t_f16; the wrappers
 * src/mxfp4.rs:242-258, src/iq2xxs.rs:396-412).  Same validation and empty case.  The
 * f32 operands live in a buffer the library keeps per stream (grown at first use, up
 * to 64 MB; larger calls take a stream-ordered allocation): with device pointers, a
 * call on a stream that has run one of its size before allocates nothing and can be
 * captured into a HIP graph, as jq_matmul_t can. */
int jq_matmul_t_f16(const jq_weight *w, size_t m, const uint16_t *lhs, size_t lhs_len, uint16_t *dst,
                    size_t dst_len, int ptrs_are_device, void *stream);

/* jq_matmul_t for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference.  Same product, same kernels, device pointers only; what jq_matmul_t
 * keeps in an allocation per stream (prepared activation operands, partial sums of a
 * product split over k) lives in one fixed array of JQ_NOALLOC_SCRATCH_BYTES in each
 * device's memory, held from library load until the process ends.  The call makes no
 * hipMalloc / hipFree and fails, dst untouched, when the product needs more scratch than
 * the array holds (one activation row never needs any; Q4_K needs about 9 KB per 16
 * activation rows and 256 columns up to 256 rows and 4 m k bytes beyond; the other
 * formats 4 m k bytes from 8 rows on; a product split over k adds 4 m n bytes a split).
 * Every call on a device shares that device's array: calls whose kernels overlap on
 * one device (two streams, two threads) race; calls on one stream are safe.
 * Where jq_matmul_t would split a product over k into more partial results than the
 * array holds, this call takes fewer splits: the result then differs from jq_matmul_t's
 * in the order of its f32 additions (within the accuracy bound, not bit for bit). */
#define JQ_NOALLOC_SCRATCH_BYTES (32u << 20)
int jq_matmul_t_noalloc(const jq_weight *w, size_t m, const float *lhs_dev, size_t lhs_len,
                        float *dst_dev, size_t dst_len, void *stream);

/* The free-function form over raw device-resident block bytes: runs the fused
 * kernel for `ggml_type` or declines (returns 1, dst untouched) when the type
 * has no kernel or nbytes is not a whole number of blocks
 * (reference: src/kquant_dot.rs:126-143 try_matmul_fused). */
int jq_try_matmul_fused(uint32_t ggml_type, size_t m, size_t k, size_t n, const float *lhs_dev,
                        const void *blocks_dev, size_t nbytes, float *dst_dev, void *stream);

/* Canonical decode of the whole weight to f32, out_len == n*k
 * (reference: src/mmap_tensor.rs:169-173 dequantize,
 * src/quant_matmul.rs:36-103 decode_raw_to_f32). */
int jq_dequantize(const jq_weight *w, float *out, size_t out_len, int out_is_device, void *stream);

/* Frees the scratch memory the library keeps for `stream` on the current device (the buffer the products
 * with prepared activations share, and every smaller one it outgrew), after waiting for the stream.  For
 * teardown: a HIP graph captured on the stream names those buffers and must not be replayed afterwards, and no
 * other thread may have a call in progress on that stream.  No
 * counterpart in the reference (its scratch is host memory owned by each call). */
int jq_stream_release(void *stream);

/* Raw tensor bytes of ggml type `ggml_type` to `elems` f32 values: every block format of this library, F16
 * (1), Q8_1 (9) and Q8_K (15).  Returns 0 with `out` filled; 2 where the reference answers Ok(None) -- F32 (0),
 * whose bytes the caller's own reader keeps exact, and every type without a decoder there; 1 with a message
 * when nbytes does not hold elems elements (the reference's wording)
 * (reference: src/quant_matmul.rs:36-103 decode_raw_to_f32). */
int jq_decode_raw_to_f32(uint32_t ggml_type, const void *bytes, size_t nbytes, size_t elems, float *out,
                         int ptrs_are_device, void *stream);

/* Row gather with decode: out[i, :] = decode(W[ids[i], :]); an id >= n fails
 * (reference: src/mmap_tensor.rs:140-167 embedding). */
int jq_embedding(const jq_weight *w, const uint32_t *ids, size_t n_ids, float *out, size_t out_len,
                 int ptrs_are_device, void *stream);

/* ---- Mixture-of-experts layer -------------------------------------------------
 * One call per layer instead of one per expert matmul: router, gating, top-k,
 * expert SwiGLU MLPs over the routed pairs grouped by expert id, weighted sum,
 * optional shared expert.  Semantics follow the reference's two MoE blocks
 * (reference: src/quantized_qwen3_moe.rs:404-528 Moe::{forward,route,dispatch,
 * dispatch_decode}; src/quantized_deepseek2.rs:508-685 with sigmoid gating,
 * selection bias, group-limited top-k, weight scale and shared expert). */
typedef struct jq_moe jq_moe;

typedef struct {
    uint32_t n_expert;       /* routed experts E */
    uint32_t n_expert_used;  /* k */
    uint32_t hidden;         /* h */
    uint32_t inter;          /* expert feed-forward length */
    uint32_t gating;         /* 0 softmax, 1 sigmoid (src/quantized_deepseek2.rs:529-532) */
    uint32_t norm_topk;      /* divide the k weights by max(sum, 6.103515625e-5) */
    float weights_scale;     /* 0 or 1: none (src/quantized_deepseek2.rs:549-551) */
    uint32_t n_group;        /* <= 1: no group limit (src/quantized_deepseek2.rs:563-566) */
    uint32_t topk_group;
    /* Clamp in front of the experts' SwiGLU: gate to (-inf, c], up to [-c, c]; <= 0: none.  The shared
     * expert has a limit of its own (src/quantized_deepseek4.rs:445-462, :2419-2448). */
    float swiglu_clamp;
    float swiglu_clamp_shared;
} jq_moe_config;

/* router_w is [E, h] row-major f32 on the host (ffn_gate_inp), router_bias [E]
 * or NULL (exp_probs_b).  gate_exps / up_exps are stacked [E*inter, h] weights,
 * down_exps [E*h, inter]; expert e is the e-th slice
 * (reference: src/quantized_qwen3_moe.rs:659-667 load_moe).  The shared expert's
 * three weights may be NULL.  The weights must outlive the layer object. */
int jq_moe_create(const jq_moe_config *cfg, const float *router_w, const float *router_bias,
                  const jq_weight *gate_exps, const jq_weight *up_exps, const jq_weight *down_exps,
                  const jq_weight *shared_gate, const jq_weight *shared_up, const jq_weight *shared_down,
                  jq_moe **out);
void jq_moe_free(jq_moe *moe);

/* Router only: ids[t, s] (descending score) and weights[t, s], s < k
 * (reference: src/quantized_qwen3_moe.rs:424-436 route). */
int jq_moe_route(jq_moe *moe, size_t n_tokens, const float *x, uint32_t *ids, float *weights,
                 int ptrs_are_device, void *stream);

/* y[n_tokens, h] = MoE(x[n_tokens, h]).  One call at a time per jq_moe (it owns
 * its scratch buffers).  Accuracy as for jq_matmul_t, with the expert matmuls' inputs
 * (x, and silu(gate) * up for the down projection) in 16-bit fixed point: one scale
 * per 32 elements on the integer-dot kernels, per 256 on the grouped GEMM.  The error
 * grows with a row's largest magnitude: measured at 8192 columns with gate and up
 * results of standard deviation 1.8 (activations up to 50, outputs up to 40), the
 * mean error is 6e-5 of max(|ref|, 1) on the integer-dot kernels and 1.4e-4 on the
 * grouped GEMM, which then passes 1e-3 on 0.3 % of the elements (largest 2.7e-3);
 * with inputs of the magnitude a normed layer gives the bound holds on every path. */
int jq_moe_forward(jq_moe *moe, size_t n_tokens, const float *x, float *y, int ptrs_are_device, void *stream);

/* ---- Multi-head latent attention (DeepSeek-V2 / V3 / Kimi-K2) -----------------------
 * The attention block of the reference's `deepseek2` graph: Q projection (plain or
 * low-rank a -> RMSNorm -> b), compressed KV projection, interleaved RoPE (YaRN-aware) on
 * the rope slices, KV up-projection, causal softmax attention over the cache, output
 * projection (reference: src/quantized_deepseek2.rs:357-499 Attention::forward,
 * :240-311 RotaryEmbedding, :875-889 the causal mask).  Results match the reference's
 * unabsorbed computation within f32 tolerance; the cache holds the normed latent and
 * the rotated shared key of every token instead of per-head keys and values. */
typedef struct jq_mla jq_mla;

typedef struct {
    uint32_t n_embd, n_head;
    uint32_t q_lora_rank;            /* 0: plain Q projection (src/quantized_deepseek2.rs:357-371) */
    uint32_t kv_lora_rank, qk_nope_head_dim, qk_rope_head_dim, v_head_dim;
    uint32_t n_ctx;                  /* positions of the cache and of the rotary tables */
    float rms_eps, rope_theta;
    /* YaRN (src/quantized_deepseek2.rs:161-192, :246-301): factor 0 = none.  The softmax
     * scale is 1/sqrt(qk_nope + qk_rope), times mscale^2 under YaRN. */
    float yarn_factor, yarn_mscale_all_dim;
    uint32_t yarn_orig_context_length;
} jq_mla_config;

/* q_or_q_a: attn_q [n_head*(nope+rope), n_embd], or attn_q_a [q_lora_rank, n_embd] with
 * q_a_norm [q_lora_rank] (host f32) and q_b = attn_q_b [n_head*(nope+rope), q_lora_rank].
 * kv_a_mqa [kv_lora_rank + rope, n_embd]; kv_a_norm [kv_lora_rank] (host f32).  The KV
 * up-projection [n_head*(nope+v), kv_lora_rank] comes as a quantized weight (kv_b) or as
 * dense row-major f32 on the host (kv_b_dense; what the reference rebuilds from the
 * pre-split attn_k_b / attn_v_b tensors, src/quantized_deepseek2.rs:931-958): exactly one
 * of the two.  o_proj [n_embd, n_head*v].  The weights must outlive the object. */
int jq_mla_create(const jq_mla_config *cfg, const jq_weight *q_or_q_a, const float *q_a_norm,
                  const jq_weight *q_b, const jq_weight *kv_a_mqa, const float *kv_a_norm,
                  const jq_weight *kv_b, const float *kv_b_dense, const jq_weight *o_proj, jq_mla **out);
void jq_mla_free(jq_mla *mla);

/* out[n_tokens, n_embd] = attention(x[n_tokens, n_embd]) for tokens at cache positions
 * pos .. pos + n_tokens - 1; `pos` must equal the number of tokens cached so far (the
 * reference appends to its cache on every call, src/quantized_deepseek2.rs:479-486).
 * Token i attends to positions 0 .. pos + i.  One call at a time per object. */
int jq_mla_forward(jq_mla *mla, size_t n_tokens, size_t pos, const float *x, float *out,
                   int ptrs_are_device, void *stream);
/* Empties the cache (reference: src/quantized_deepseek2.rs:501-503 clear_kv_cache). */
int jq_mla_reset(jq_mla *mla);
/* Tokens in the cache. */
size_t jq_mla_cached_tokens(const jq_mla *mla);

/* ---- Dense Qwen3 decoder (end-to-end decode harness) -----------------------------
 * The graph the reference runs for a qwen3 GGUF: embedding gather, per layer
 * RMSNorm -> q/k/v -> per-head q/k RMSNorm -> half-split RoPE -> KV append ->
 * causal GQA attention -> o + residual -> RMSNorm -> SwiGLU MLP + residual,
 * then the last position's output norm and logits
 * (reference: src/embedding.rs:297-396 for the layer, src/quantized_qwen3_moe.rs:
 * 231-386,776-819 for attention, RoPE, KV cache and last-token logits;
 * src/engine.rs:1149-1294 for the prefill-then-one-token-per-step contract). */
typedef struct jq_model jq_model;

typedef struct {
    uint32_t n_layer, hidden, n_head, n_kv_head, head_dim, ffn, vocab, n_ctx;
    float rms_eps, rope_theta;
    /* Qwen3-MoE (general.architecture = qwen3moe; reference: src/quantized_qwen3_moe.rs:100-147):
     * n_expert > 0 makes every layer's feed-forward block a mixture of experts (softmax over all
     * experts, top n_expert_used, weights divided by their sum when norm_topk_prob), ffn is then
     * unused and may be 0.  All four zero: the dense model. */
    uint32_t n_expert, n_expert_used, expert_ffn, norm_topk_prob;
} jq_qwen3_config;

int jq_qwen3_create(const jq_qwen3_config *cfg, jq_model **out);
void jq_qwen3_free(jq_model *model);

/* The configuration the model was created with (for models built by jq_qwen3_load_gguf). */
int jq_qwen3_get_config(const jq_model *model, jq_qwen3_config *out);

/* Installs one tensor under its GGUF name ("token_embd.weight",
 * "blk.3.attn_q.weight", "blk.3.attn_q_norm.weight", "output_norm.weight",
 * "output.weight", ...).  ggml_type 0 is F32 (norm weights); the others are the
 * JQ_TYPE_* ids, uploaded in native block layout.  The expected shape comes
 * from the configuration; a wrong byte count fails.  A mixture-of-experts model
 * takes "blk.N.ffn_gate_inp.weight" (F32 or F16, [n_expert, hidden]) and the stacked
 * "blk.N.ffn_{gate,up,down}_exps.weight" ([n_expert, out, in], expert e the e-th
 * slice; reference: src/quantized_qwen3_moe.rs:556-571, :653-675) in place of the
 * dense ffn_gate / ffn_up / ffn_down. */
int jq_qwen3_set_tensor(jq_model *model, const char *name, uint32_t ggml_type, const void *data,
                        size_t nbytes);

/* Appends n_tokens tokens at absolute position pos (which must equal the number
 * of tokens fed so far) and writes vocab logits for the last one
 * (the contract of the reference's plugin ABI, src/npu/mod.rs:44-50).  tokens is
 * a host pointer; logits goes to host or device memory. */
int jq_qwen3_forward(jq_model *model, const uint32_t *tokens, uint32_t n_tokens, uint32_t pos,
                     float *logits, int logits_on_device, void *stream);

/* Greedy pick over the logits of the last forward: the LAST index holding the
 * maximum, as the reference's sampler does (src/engine.rs:2371-2378). */
int jq_qwen3_greedy(jq_model *model, uint32_t *token, void *stream);

/* Forgets the KV cache (reference: clear_kv_cache, src/quantized_qwen3_moe.rs:822-826). */
int jq_qwen3_reset(jq_model *model);

/* ---- GGUF files -------------------------------------------------------------------
 * A tolerant reader of the container: header, metadata and tensor directory of a
 * file mapped read-only, tensor types kept as raw ids so that MXFP4 (39) and
 * IQ2_XXS (16) survive parsing (reference: src/gguf_ext.rs:400-480 read_header with
 * the limits of :33-59; the mapping and its bounds check src/mmap_tensor.rs:105-123).
 * Host only: none of the jq_gguf_* calls except jq_gguf_upload touches the GPU. */
typedef struct jq_gguf jq_gguf;

/* Bytes of `elems` elements of a raw type id, for every id the reference sizes
 * (F32, F16, BF16, Q4_0..Q8_1, Q2_K..Q8_K, I32, IQ2_XXS, MXFP4); fails for an
 * unknown id or a count that is not whole blocks
 * (reference: src/gguf_ext.rs:483-512 type_size_bytes). */
int jq_type_size_bytes(uint32_t ggml_type, size_t elems, size_t *bytes);

/* Maps `path` and parses its header. */
int jq_gguf_open(const char *path, jq_gguf **out);
/* Parses a header held in memory (the bytes are copied); tensor data may be absent. */
int jq_gguf_parse(const void *bytes, size_t len, jq_gguf **out);
void jq_gguf_close(jq_gguf *g);

uint32_t jq_gguf_version(const jq_gguf *g);
uint64_t jq_gguf_tensor_data_offset(const jq_gguf *g);
size_t jq_gguf_tensor_count(const jq_gguf *g);
size_t jq_gguf_metadata_count(const jq_gguf *g);

/* Directory entry `index` (file order).  dims has room for 8 values and receives them
 * in row-major order, slowest first (the file stores them fastest first); offset counts
 * from jq_gguf_tensor_data_offset.  Any output pointer may be NULL.  `*name` stays
 * valid until jq_gguf_close (reference: src/gguf_ext.rs:117-135 RawTensorInfo). */
int jq_gguf_tensor_at(const jq_gguf *g, size_t index, const char **name, uint32_t *ggml_type, uint32_t *n_dims,
                      uint64_t *dims, uint64_t *offset);
int jq_gguf_find_tensor(const jq_gguf *g, const char *name, size_t *index);
/* The tensor's bytes inside the mapping; fails when its type has no known size or the
 * range runs past the end of the file. */
int jq_gguf_tensor_bytes(const jq_gguf *g, size_t index, const void **data, size_t *nbytes);

/* Metadata scalars: nonzero when the key is missing or holds another type.  u32 accepts
 * every integer type up to 32 bits that is not negative
 * (reference: src/quantized_qwen3_moe.rs:64-88 Meta helpers). */
int jq_gguf_meta_u32(const jq_gguf *g, const char *key, uint32_t *out);
int jq_gguf_meta_f32(const jq_gguf *g, const char *key, float *out);
int jq_gguf_meta_bool(const jq_gguf *g, const char *key, int *out);
int jq_gguf_meta_str(const jq_gguf *g, const char *key, const char **out, size_t *len);
int jq_gguf_meta_array_len(const jq_gguf *g, const char *key, size_t *len);

/* Uploads one tensor once, in its native block layout, straight from the mapping: a
 * matrix [n, k], or a stack [E, n, k] as one weight of E*n rows whose expert slices
 * jq_view addresses (reference: src/mmap_tensor.rs:520-565 borrowed_qtensor_raw,
 * src/quantized_qwen3_moe.rs:596-631 split_experts). */
int jq_gguf_upload(const jq_gguf *g, const char *name, jq_weight **out);

/* Builds a Qwen3 decoder from a GGUF file, dense (general.architecture = qwen3) or
 * mixture-of-experts (qwen3moe: expert_count, expert_used_count and
 * expert_feed_forward_length required, attention.norm_topk_prob defaulting to true,
 * expert tensors shaped [n_expert, out, in]): configuration from the `<arch>.*`
 * metadata with the reference loader's rules (attention.key_length wins over
 * embedding_length / head_count, rope.freq_base defaults to 10000; reference:
 * src/quantized_qwen3_moe.rs:90-147), every tensor uploaded once; a file without
 * output.weight uses token_embd.weight as the output head
 * (reference: src/quantized_qwen3_moe.rs:737-743).  n_ctx == 0 takes the file's
 * context_length. */
int jq_qwen3_load_gguf(const char *path, uint32_t n_ctx, jq_model **out);

/* ---- Model-level plugin boundary ----------------------------------------------------
 * The four symbols the reference engine looks up when it is started with a backend
 * library (reference: src/npu/mod.rs:32-50 contract; src/npu/vendor.rs:17-20
 * signatures, :49-56 symbol check, :95-121 init; src/main.rs:166-172 the switch).
 * init loads the GGUF at model_path as a dense Qwen3 decoder with a KV cache of
 * n_ctx tokens and reports the vocabulary size; forward appends n_tokens tokens at
 * absolute position pos, which must equal the number of tokens fed so far, and
 * writes vocab logits for the last one; reset forgets the fed tokens.  0 is success;
 * the codes are those of the reference's model plugin
 * (crates/joshua-mock-npu/src/lib.rs:41-131): -1 null argument or empty batch,
 * -2 the model did not load, -3 pos is not the number of tokens fed so far,
 * -4 the context is full, -5 the device call failed (jq_last_error has the text).
 * A handle is used by one thread at a time but may move between threads. */
int32_t joshua_npu_init(const char *model_path, uint32_t n_ctx, uint32_t *out_vocab, void **out_handle);
int32_t joshua_npu_forward(void *handle, const uint32_t *tokens, uint32_t n_tokens, uint32_t pos,
                           float *out_logits);
int32_t joshua_npu_reset(void *handle);
void joshua_npu_free(void *handle);

/* Blocks until everything enqueued on `stream` has finished. */
int jq_stream_synchronize(void *stream);

#ifdef __cplusplus
}
#endif
#endif
