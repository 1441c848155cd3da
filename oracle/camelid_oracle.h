/*
 * camelid_oracle.h -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A scalar CPU restatement, in plain C, of the reference engine's quantized
 * weight-times-activation path (GGUF Q8_0 / Q4_0 / Q4_K / Q6_K weights against
 * Q8_0 / Q8_K quantized activations).  It exists so that the HIP kernels can be
 * compared against the reference arithmetic on the same seeded inputs, and so
 * that the benchmark can time "the reference CPU path, restated" on the host
 * cores of the GPU box.  Nothing in the shipped library links or calls this.
 *
 * Every function cites the reference file:line (paths under the reference
 * checkout) whose arithmetic it follows, operation for operation.  Build with
 * -ffp-contract=off: the reference's generic-order dots round every multiply
 * and add separately; the places where the reference fuses (`mul_add`) call
 * fmaf() explicitly.
 *
 * Pinning status (what independent evidence holds each function in place):
 *   f16 <-> f32                : F16 golden fixture (gguf 0.19.0 bit patterns),
 *                                exhaustive cross-check against numpy float16.
 *   dequant Q8_0/Q4_0/Q4_K/Q6_K: golden fixtures under tests/golden/dequant
 *                                (bit patterns, zero tolerance).
 *   quantize_q8_0 / q8_k       : known answers from the reference's unit tests,
 *                                tie cases, closed forms, numpy restatement.
 *   integer block dots         : brute force over dequantized integers.
 *   row dots (final f32)       : f64 dot of the fixture-pinned dequant output
 *                                against dequantized activations (the reference
 *                                tests' own criterion), cross-variant agreement.
 *                                The *bitwise* value of the final f32 has no
 *                                stored vector in the reference; its association
 *                                is held by an independent evaluator instead
 *                                (tests/test_oracle_association.py: integers from
 *                                the numpy decoders, every float step in exact
 *                                rationals with an explicit round to binary32),
 *                                on inputs where the plausible wrong orders give
 *                                other bits.  What stays transcription: that the
 *                                formula written into that evaluator is the one
 *                                in the Rust source.
 *   softmax_top_k, router_     : closed forms and brute force on small inputs;
 *   softmax_top_k                libm expf may differ from Rust's by 1 ulp.
 *   gelu_tanh_mul, silu_mul    : f64 evaluation of the formula within 1e-6; libm
 *                                tanhf / expf vs Rust's: last ulp unpinned.
 *   rms_norm                   : the reference's known vector (tests/
 *                                tensor_primitives.rs:83-93), exact power-of-two
 *                                cases, an order-sensitive input checked against
 *                                an independent sequential sum, f64 within 1e-6.
 *   weight quantizers          : reconstruction-error bounds on the reference's
 *                                ramps; they only generate inputs.
 */
#ifndef CAMELID_ORACLE_H
#define CAMELID_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GGUF tensor type ids (reference src/gguf/reader.rs:94-127). */
enum {
    ORC_Q4_0 = 2,
    ORC_Q8_0 = 8,
    ORC_Q4_K = 12,
    ORC_Q6_K = 14
};

/* Accumulation orders that exist in the reference for the K-quants. */
enum {
    ORC_ORDER_PRIMARY = 0, /* Q4_K: fused single chain (q4_k_dot_arm); Q6_K: 8-lane; Q8_0/Q4_0: block order */
    ORC_ORDER_ALT = 1      /* Q4_K: generic 8-lane (q4_k_wire_row_dot); Q6_K: fused single chain (q6_k_dot_arm) */
};

int orc_block_values(int fmt);
int orc_block_bytes(int fmt);

/* f16 conversion: src/inference.rs:27062-27125. */
uint16_t orc_f32_to_f16_bits(float v);
float orc_f16_bits_to_f32(uint16_t h);
void orc_f32_to_f16_bits_array(const float *v, size_t n, uint16_t *out);
void orc_f16_bits_to_f32_array(const uint16_t *h, size_t n, float *out);

/* Activation quantizers. */
/* src/inference.rs:22510-22528 (one scale + 32 int8 per block). */
void orc_quantize_q8_0(const float *x, size_t n, float *scales, int8_t *q);
/* src/inference.rs:23112-23152 (one d + 256 int8 per super-block). */
void orc_quantize_q8_k(const float *x, size_t n, float *d, int8_t *q);

/* Weight dequantizers (bit-exact targets). n_blocks blocks of wire bytes -> f32. */
void orc_dequant(int fmt, const uint8_t *wire, size_t n_blocks, float *out);

/* Row dots: one weight row (wire bytes) against one quantized activation row. */
float orc_q8_0_row_dot(const uint8_t *w, const float *xs, const int8_t *xq, size_t n_blocks);
float orc_q4_0_row_dot(const uint8_t *w, const float *xs, const int8_t *xq, size_t n_blocks);
float orc_q4_k_row_dot_arm(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb);
float orc_q4_k_row_dot_generic(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb);
float orc_q6_k_row_dot_lanes(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb);
float orc_q6_k_row_dot_arm(const uint8_t *w, const float *xd, const int8_t *xq, size_t n_sb);

/*
 * Exact per-block integers of one row (the quantities every reference variant
 * agrees on).  Q8_0/Q4_0: out[b] = isum of block b (1 int per block).
 * Q4_K: out[2*i] = sum_g sc_g * dot_g ("sumi1+sumi2"), out[2*i+1] = sum_g
 * bsum32_g * m_g ("prod" / "sumi").  Q6_K: out[i] = sum_j sc_j * dot16_j with
 * the -32 bias applied (sum of the 8 aux32 lanes).
 */
void orc_row_block_ints(int fmt, const uint8_t *w, const int8_t *xq, size_t n_blocks, int32_t *out);

/*
 * Drivers (src/gemma4_runtime.rs:826-1150): quantize each activation row once,
 * then one row dot per (token, output row).  out is token-major:
 * out[t * rows + o].  rows are taken from row_start (expert band).  threads<=1
 * runs serially; otherwise output rows are handed out in chunks of 64 rows
 * (ROW_CHUNK) to `threads` pthreads.
 */
int orc_matmul(int fmt, int order, const uint8_t *wire, size_t cols,
               size_t row_start, size_t rows,
               const float *x, size_t n_tokens, float *out, int threads);

/* Same, but against already quantized activations (scales: per 32 for the
 * Q8_0 family, per 256 for the K family). */
int orc_matmul_q(int fmt, int order, const uint8_t *wire, size_t cols,
                 size_t row_start, size_t rows,
                 const float *xscales, const int8_t *xq, size_t n_tokens,
                 float *out, int threads);

/* Mixtral routing: src/inference.rs:13940-13991.  Writes min(k, n) pairs,
 * returns the count. */
int orc_softmax_top_k(const float *logits, int n, int k, int32_t *idx, float *w);

/* Gemma-4 routing (src/gemma4_runtime.rs:61-84, :5567-5610): softmax over all experts, top-k by
 * probability (ties to the lower index), scale[s] = down_scale[e] * (p[e] / max(sum selected, 6.103515e-5));
 * down_scale may be NULL (= 1).  Returns the count written. */
int orc_router_softmax_top_k(const float *logits, int n, int k, const float *down_scale, int32_t *idx, float *scale);

/* gelu_pytorch_tanh(a) * b: src/gemma4_mtp.rs:172-175, src/gemma4_runtime.rs:5689-5691. */
void orc_gelu_tanh_mul(const float *a, const float *b, size_t n, float *out);

/* RMS norm, the step upstream of the activation quantizers:
 * src/tensor/mod.rs:2707-2760 (sequential f32 sum of squares). */
void orc_rms_norm(const float *x, const float *weight, float eps, size_t rows, size_t cols, float *out);

/* Expert activation: src/tensor/mod.rs:2610-2634. */
void orc_silu_mul(const float *a, const float *b, size_t n, float *out);

/*
 * Mixture-of-experts FFN for quantized expert matrices, composed from the
 * pieces above in the order src/inference.rs:14142-14280 applies them:
 * route, then per selected expert (in routed order) gate/up matvec, silu_mul,
 * down matvec, out += y * weight.  gate/up/down hold n_experts matrices back
 * to back (expert e = rows e*ff.. of gate/up, rows e*hidden.. of down).
 * logits: [n_tokens][n_experts]; x, out: [n_tokens][hidden].
 */
int orc_moe_ffn(int fmt, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                int n_experts, int top_k, size_t hidden, size_t ff,
                const float *logits, const float *x, size_t n_tokens,
                float *out, int threads);

/* The same with the routing / activation variant spelled out: variant 0 = Mixtral as above,
 * 1 = Gemma-4 (orc_router_softmax_top_k with down_scale, gelu_tanh).  up == NULL: `gate` holds
 * fused gate|up experts of 2*ff rows each. */
int orc_moe_ffn_ex(int fmt, int fmt_down, const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                   int n_experts, int top_k, size_t hidden, size_t ff,
                   const float *logits, const float *x, size_t n_tokens,
                   float *out, int threads, int variant, const float *down_scale);

/* Weight quantizers used to make synthetic inputs: src/quantize.rs:98-244.
 * Q6_K has no quantizer in the reference; orc_quantize_weights builds Q6_K
 * super-blocks with a ggml-style search-free scheme of its own (inputs only). */
int orc_quantize_weights(int fmt, const float *src, size_t n, uint8_t *dst, int threads);

#ifdef __cplusplus
}
#endif
#endif
