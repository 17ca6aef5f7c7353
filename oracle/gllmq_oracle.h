/*
 * CPU oracle for the quantized-weight matmul path of putao520/gllm.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check
 * and the cpu_baseline leg of bench.py may load it; the product path
 * (gllm_amd/, libgllm_hip_quant.so) never links, imports or calls it.
 *
 * What it restates (all paths relative to the reference tree):
 *   - GGUF block constants ............ src/loader/gguf/types.rs:57-94,152-236,443-472
 *   - Backend::dequantize ............. src/compat/cpu_backend.rs:1051-1159
 *   - Backend::quantized_matmul ....... src/compat/cpu_backend.rs:991-1049
 *   - Q4_K / Q5_K / Q6_K codecs ....... docs/domain-knowledge/quant-kquant-iq-proprietary.md:40-64,123-154
 *                                       tests/test_diag_q5km_block_bytes.rs:13-39
 *   - Q8_0 codec ...................... docs/domain-knowledge/gguf-classic-quant-layout.md:33,46,64
 *   - MoE routing and combine ......... src/moe/routing.rs:100-173,263-327
 *
 * The arithmetic of kquant_matmul / classic_matmul / dequant_* lives in the crate
 * gllm-kernels 0.1.0 (path dependency, Cargo.toml:44, Cargo.lock:839-853), which is
 * not part of the reference tree.  The codecs are therefore restated from the
 * documents above, which themselves quote llama.cpp's dequantize_row_q*_K /
 * get_scale_min_k4, and pinned by the checks in tests/test_oracle_*.py.
 *
 * Parity status per function:
 *   gq_dequantize (Q4_K,Q5_K,Q6_K,Q8_0) : pinned (closed forms, bit walks, documented
 *                                         known answers, independent numpy twin)
 *   gq_softmax / gq_topk_with_weights /
 *   gq_route / gq_expert_capacity       : pinned by the reference's unit-test vectors
 *   gq_quantized_matmul                 : value = deq(W) . x is pinned; the reference's
 *                                         summation order, threading and any internal
 *                                         activation handling are PARITY UNPINNED (no
 *                                         test or fixture of the reference exercises it)
 *   gq_quantized_matmul_avx2 / _avx512  : the vectorised baseline flavours; decoders pinned bitwise
 *                                         against the scalar ones, the sum against the f64 yardstick;
 *                                         same status as gq_quantized_matmul otherwise
 *   gq_quant_gather                     : unscaled lookups are pinned with gq_dequantize (a row
 *                                         gather of its output); where the embedding scale is
 *                                         applied is PARITY UNPINNED (the op runs in generated
 *                                         code of gllm-kernels, no test of the reference holds
 *                                         a value)
 *   gq_argmax_token                     : pinned by the reference's unit-test vectors
 *                                         (src/engine/executor_step.rs:2191-2325)
 *   gq_ffn_swiglu                       : the formula down(silu(gate x) * (up x)) is the reference's
 *                                         (04-OPERATORS.md:114); pinned against a float64 numpy
 *                                         evaluation of it; the products inherit gq_quantized_matmul's
 *                                         status
 *   gq_moe_ffn                          : PARITY UNPINNED beyond routing + combine rule
 *                                         (the reference's quantized expert template is
 *                                         unfinished, build_graph.inc.rs:2922-2942)
 */
#ifndef GLLMQ_ORACLE_H
#define GLLMQ_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* GgmlDType ids, src/loader/gguf/types.rs:57-94 */
enum {
    GQ_TYPE_Q8_0 = 8,
    GQ_TYPE_Q4_K = 12,
    GQ_TYPE_Q5_K = 13,
    GQ_TYPE_Q6_K = 14
};

/* accumulate modes for gq_quantized_matmul */
enum {
    GQ_ACC_F32 = 0, /* reference-faithful: decode block to f32, then f32 multiply-add */
    GQ_ACC_F64 = 1  /* same products summed in double: the parity yardstick          */
};

/* return codes */
enum {
    GQ_OK = 0,
    GQ_ERR_UNIMPLEMENTED = 1,
    GQ_ERR_BAD_SHAPE = 2
};

/* elements / bytes per block; 0 for a dtype this oracle does not cover */
size_t gq_block_size(uint32_t ggml_dtype);
size_t gq_block_bytes(uint32_t ggml_dtype);
/* ceil(k / block_size) * block_bytes, tensor_nbytes rule for one row */
size_t gq_row_bytes(uint32_t ggml_dtype, size_t k);

float gq_f16_to_f32(uint16_t h);
uint16_t gq_f32_to_bf16_rne(float f);

/* sc/m pair j (0..7) of a 12-byte packed scale field */
void gq_scale_min_k4(int j, const uint8_t *scales12, uint8_t *sc, uint8_t *m);

/* One block each. */
void gq_dequant_block_q4_k(const uint8_t *blk, float *out256);
void gq_dequant_block_q5_k(const uint8_t *blk, float *out256);
void gq_dequant_block_q6_k(const uint8_t *blk, float *out256);
void gq_dequant_block_q8_0(const uint8_t *blk, float *out32);

/* Backend::dequantize: whole blocks of `blocks` paired with whole block-size chunks
 * of `out`; trailing partial chunks on either side are ignored. */
int gq_dequantize(const uint8_t *blocks, size_t n_bytes, float *out, size_t n_out,
                  uint32_t ggml_dtype);

/* Op::QuantGather (build_graph.inc.rs:203-211): out[i] = row ids[i] of the quantized table
 * (vocab rows of `hidden` elements), decoded, times `scale` when `scaled`.  GQ_ERR_BAD_SHAPE
 * for an id >= vocab. */
int gq_quant_gather(const uint8_t *table, uint32_t ggml_dtype, size_t vocab, size_t hidden,
                    const uint32_t *ids, size_t count, float scale, int scaled, float *out);

/* argmax_token (src/engine/executor_step.rs:48-55): index of the largest entry that is not
 * NaN, the last one of equal maxima; -1 when there is none. */
int64_t gq_argmax_token(const float *logits, size_t n);

/* Backend::quantized_matmul: y[m x n] = x[m x k] . W[n x k]^T, W as n rows of
 * gq_row_bytes(dtype,k) bytes.  threads <= 1 runs on the calling thread. */
int gq_quantized_matmul(const uint8_t *w, const float *x, float *y, uint32_t ggml_dtype,
                        size_t m, size_t n, size_t k, int acc_mode, int threads);

/* Same contraction with both operands rounded to bf16 (round-to-nearest-even) before
 * the multiply and products summed in double: yardstick for the MFMA path. */
int gq_quantized_matmul_bf16(const uint8_t *w, const float *x, float *y, uint32_t ggml_dtype,
                             size_t m, size_t n, size_t k, int threads);

/* The vectorised flavour of the CPU baseline: the block decoders eight elements at a time
 * (AVX2; every decoded value equal to the scalar decoder's bit for bit) and an f32 dot product
 * over eight-lane partial sums.  GQ_ERR_UNIMPLEMENTED when the build or the host has no AVX2+FMA.
 * gq_dequant_block_avx2 decodes one block with those decoders (for the bit-equality test). */
int gq_have_avx2(void);
int gq_dequant_block_avx2(uint32_t ggml_dtype, const uint8_t *blk, float *out);
int gq_quantized_matmul_avx2(const uint8_t *w, const float *x, float *y, uint32_t ggml_dtype,
                             size_t m, size_t n, size_t k, int threads);

/* The same sixteen elements at a time (AVX-512 F/BW/VL/DQ, compiled by function attribute and
 * chosen at run time): decoders again equal to the scalar ones bit for bit, the dot product over
 * sixteen-lane partial sums.  GQ_ERR_UNIMPLEMENTED where the host has no AVX-512. */
int gq_have_avx512(void);
int gq_dequant_block_avx512(uint32_t ggml_dtype, const uint8_t *blk, float *out);
int gq_quantized_matmul_avx512(const uint8_t *w, const float *x, float *y, uint32_t ggml_dtype,
                               size_t m, size_t n, size_t k, int threads);

/* src/moe/routing.rs:290-302 */
void gq_softmax(const float *logits, size_t n, float *probs);
/* src/moe/routing.rs:263-280; writes min(k,n) pairs, returns that count */
size_t gq_topk_with_weights(const float *logits, size_t n, size_t k, uint32_t *idx, float *w);
/* src/moe/routing.rs:283-287 */
size_t gq_topk_indices(const float *logits, size_t n, size_t k, uint32_t *idx);
/* src/moe/routing.rs:53-61 */
size_t gq_expert_capacity(float capacity_factor, size_t total_tokens, size_t num_experts);
/* ExpertRouteTable::from_gate_logits, src/moe/routing.rs:100-160.
 * logits [tokens x experts]; outputs are [tokens x max(top_k, 1)], route_len[t] entries valid
 * (with top_k = 0 every token still gets the least-loaded fallback, as in the reference).
 * Returns overflow_count. expert_counts [experts]. */
size_t gq_route(const float *logits, size_t tokens, size_t experts, size_t top_k,
                float capacity_factor, uint32_t *route_expert, float *route_weight,
                uint32_t *route_pos, uint32_t *route_len, uint32_t *expert_counts);

/* MoE expert FFN over a routing table:
 *   out[t] = sum_i w_i * down_e( act(gate_e x_t) * (up_e x_t) ),  e = route_expert[t][i]
 * gate_up: per expert 2*ffn rows of dtype_gu over hidden (gate rows first, then up rows);
 * down:    per expert hidden rows of dtype_dn over ffn.
 * relu_gate != 0 applies max(g,0) before silu (BUG-KNOWLEDGE.md:1434-1440). */
/* Dense feed-forward block: out[m x hidden] = (silu(x . gate^T) * (x . up^T)) . down^T; gate and up
 * are [ffn x hidden] of dtype_gu, down is [hidden x ffn] of dtype_dn; relu_gate: ReLU ahead of the SiLU. */
int gq_ffn_swiglu(const uint8_t *gate, const uint8_t *up, uint32_t dtype_gu, const uint8_t *down, uint32_t dtype_dn,
                  const float *x, float *out, size_t m, size_t hidden, size_t ffn, int relu_gate, int acc, int threads);

int gq_moe_ffn(const uint8_t *gate_up, uint32_t dtype_gu, const uint8_t *down, uint32_t dtype_dn,
               const float *x, float *out, size_t tokens, size_t hidden, size_t ffn,
               size_t experts, size_t top_k, const uint32_t *route_expert,
               const float *route_weight, const uint32_t *route_len, int relu_gate,
               int acc_mode, int threads);

#ifdef __cplusplus
}
#endif
#endif
