// C++ host mirror of the reference's backend interface for the quantized-weight matmul path,
// on top of the C ABI in gllm_hip_quant.h.  Header-only; link with libgllm_hip_quant.so.
//
// Mirrors (paths inside putao520/gllm):
//   trait Backend<E>::quantized_matmul / ::dequantize   src/compat/mod.rs:233-256
//   enum BackendError                                   src/engine/executor_types.rs:322-329
//   enum QuantType (kernel-side format names)           src/loader/adapter.rs:138-191
//   GgmlDType::{block_size, block_bytes}                src/loader/gguf/types.rs:152-236
//
// The reference's methods take host slices (`&[u8]`, `&[E]`, `&mut [E]`) and return
// `Result<(), BackendError>`; the methods below keep the names, argument order and meaning
// and return a BackendError value whose kind is None on success.  Device-resident forms
// (`*_device`) take HIP device pointers and a stream and are the ones a GPU executor uses:
// weights are uploaded once (src/compat/hip_backend.rs:141-156) and stay put.
#ifndef GLLM_HIP_QUANT_HPP
#define GLLM_HIP_QUANT_HPP

#include <cstddef>
#include <cstdint>
#include <string>
#include <vector>

#include "gllm_hip_quant.h"

namespace gllm {

// Names follow QuantType of the reference; values are the GGUF type ids.
enum class QuantType : uint32_t {
    Q4_0 = 2, Q4_1 = 3, Q5_0 = 6, Q5_1 = 7, Q8_0 = 8, Q8_1 = 9,
    Q2K = 10, Q3K = 11, Q4K = 12, Q5K = 13, Q6K = 14, Q8K = 15,
};

struct BackendError {
    enum class Kind { None, Hip, Unimplemented, Other };
    Kind kind = Kind::None;
    std::string message;
    bool ok() const { return kind == Kind::None; }
    explicit operator bool() const { return !ok(); } // true when an error is held
};

inline size_t block_size(QuantType t) { return gllmq_block_size(static_cast<uint32_t>(t)); }
inline size_t block_bytes(QuantType t) { return gllmq_block_bytes(static_cast<uint32_t>(t)); }
inline size_t row_bytes(QuantType t, size_t k) { return gllmq_row_bytes(static_cast<uint32_t>(t), k); }

class HipBackend {
public:
    explicit HipBackend(int device = 0)
    {
        const int rc = gllmq_init(&ctx_, device);
        if (rc != GLLMQ_OK) {
            ctx_ = nullptr;
            init_error_ = make(rc, "gllmq_init");
        }
    }
    ~HipBackend() { gllmq_destroy(ctx_); }
    HipBackend(const HipBackend &) = delete;
    HipBackend &operator=(const HipBackend &) = delete;

    const BackendError &init_error() const { return init_error_; }

    // fn quantized_matmul(&self, weight_blocks, input, output, quant_type, m, n, k)
    BackendError quantized_matmul(const uint8_t *weight_blocks, size_t weight_len, const float *input, size_t input_len,
                                  float *output, size_t output_len, QuantType quant_type, size_t m, size_t n,
                                  size_t k) const
    {
        if (!ctx_) return init_error_;
        if (input_len < m * k || output_len < m * n)
            return BackendError{ BackendError::Kind::Other, "quantized_matmul: input/output shorter than m*k / m*n" };
        return make(gllmq_quantized_matmul_host(ctx_, weight_blocks, weight_len, input, output,
                                                static_cast<uint32_t>(quant_type), m, n, k),
                    "quantized_matmul");
    }

    // fn dequantize(&self, block_data, output, quant_type)
    BackendError dequantize(const uint8_t *block_data, size_t block_len, float *output, size_t output_len,
                            QuantType quant_type) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_dequantize_host(ctx_, block_data, block_len, output, output_len,
                                          static_cast<uint32_t>(quant_type)),
                    "dequantize");
    }

    // Device-resident forms: all pointers are HIP device addresses, `stream` a hipStream_t.
    BackendError quantized_matmul_device(const void *w_dev, size_t w_bytes, const float *x_dev, float *y_dev,
                                         QuantType quant_type, size_t m, size_t n, size_t k, void *stream = nullptr,
                                         int act_mode = GLLMQ_ACT_F32_SPLIT) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_quantized_matmul_ex(ctx_, w_dev, w_bytes, x_dev, y_dev, static_cast<uint32_t>(quant_type), m,
                                              n, k, act_mode, stream),
                    "quantized_matmul");
    }

    BackendError dequantize_device(const void *blocks_dev, size_t n_bytes, float *out_dev, size_t n_out,
                                   QuantType quant_type, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_dequantize(ctx_, blocks_dev, n_bytes, out_dev, n_out, static_cast<uint32_t>(quant_type),
                                     stream),
                    "dequantize");
    }

    BackendError quantized_matmul_batch_device(const gllmq_matmul_desc *descs, size_t count,
                                               void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_quantized_matmul_batch(ctx_, descs, count, stream), "quantized_matmul_batch");
    }

    // Op::QuantGather over host slices (table uploaded, rows downloaded); ids outside the table
    // are an error of kind Other here, since the host can see them.
    BackendError quant_gather(const uint8_t *table, size_t table_len, QuantType quant_type, size_t vocab_size,
                              size_t hidden_dim, const uint32_t *token_ids, size_t count, const float *scale,
                              float *output, size_t output_len) const
    {
        if (!ctx_) return init_error_;
        if (output_len < count * hidden_dim)
            return BackendError{ BackendError::Kind::Other, "quant_gather: output shorter than count * hidden_dim" };
        return make(gllmq_quant_gather_host(ctx_, table, table_len, static_cast<uint32_t>(quant_type), vocab_size,
                                            hidden_dim, token_ids, count, scale ? *scale : 1.0f, output),
                    "quant_gather");
    }

    // Op::QuantGather { quant_type, vocab_size, hidden_dim, scale } over device buffers
    // (src/arch/auto_graph_fragments/build_graph.inc.rs:203-211); scale = nullptr: none.
    BackendError quant_gather_device(const void *table_dev, size_t table_bytes, QuantType quant_type, size_t vocab_size,
                                     size_t hidden_dim, const uint32_t *token_ids_dev, size_t count, const float *scale,
                                     float *out_dev, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_quant_gather(ctx_, table_dev, table_bytes, static_cast<uint32_t>(quant_type), vocab_size,
                                       hidden_dim, token_ids_dev, count, scale ? *scale : 1.0f, out_dev, stream),
                    "quant_gather");
    }

    // Op::QuantGather into rows of element type `elem` (GLLMQ_ELEM_*): the f32 lookup's values,
    // rounded to nearest even by the lookup's own stores.
    BackendError quant_gather_elem_device(const void *table_dev, size_t table_bytes, QuantType quant_type,
                                          size_t vocab_size, size_t hidden_dim, const uint32_t *token_ids_dev, size_t count,
                                          const float *scale, void *out_dev, int elem, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_quant_gather_elem(ctx_, table_dev, table_bytes, static_cast<uint32_t>(quant_type), vocab_size,
                                            hidden_dim, token_ids_dev, count, scale ? *scale : 1.0f, out_dev, elem, stream),
                    "quant_gather");
    }

    // Dense feed-forward block over device buffers: gate_proj, up_proj, Op::SwiGlu, down_proj
    // (src/arch/auto_graph_fragments/build_graph.inc.rs:1957-1995).
    BackendError ffn_swiglu_device(const void *gate_dev, const void *up_dev, size_t gate_up_bytes_each, QuantType t_gate_up,
                                   const void *down_dev, size_t down_bytes, QuantType t_down, const float *x_dev,
                                   float *out_dev, size_t m, size_t hidden, size_t ffn, bool relu_gate = false,
                                   void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_ffn_swiglu(ctx_, gate_dev, up_dev, gate_up_bytes_each, static_cast<uint32_t>(t_gate_up), down_dev,
                                     down_bytes, static_cast<uint32_t>(t_down), x_dev, out_dev, m, hidden, ffn,
                                     relu_gate ? 1 : 0, stream),
                    "ffn_swiglu");
    }

    // The same for E = f32 / f16 / bf16 activations and outputs (`elem`: GLLMQ_ELEM_*), replacing
    // out_dev or, with accumulate, added to it (Op::Add of a shared expert's block and the
    // residual, build_graph.inc.rs:2132-2170); one rounding to nearest even.
    BackendError ffn_swiglu_elem_device(const void *gate_dev, const void *up_dev, size_t gate_up_bytes_each,
                                        QuantType t_gate_up, const void *down_dev, size_t down_bytes, QuantType t_down,
                                        const void *x_dev, void *out_dev, size_t m, size_t hidden, size_t ffn, int elem,
                                        bool accumulate = false, bool relu_gate = false, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_ffn_swiglu_elem(ctx_, gate_dev, up_dev, gate_up_bytes_each, static_cast<uint32_t>(t_gate_up),
                                          down_dev, down_bytes, static_cast<uint32_t>(t_down), x_dev, out_dev, m, hidden, ffn,
                                          relu_gate ? 1 : 0, elem, accumulate ? GLLMQ_OUT_ACCUMULATE : 0, stream),
                    "ffn_swiglu");
    }

    // Op::Argmax over device logits [rows][ld] (argmax_token, src/engine/executor_step.rs:48-55).
    BackendError argmax_device(const float *logits_dev, size_t rows, size_t n, size_t ld, uint32_t *token_dev,
                               float *value_dev = nullptr, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_argmax(ctx_, logits_dev, rows, n, ld, token_dev, value_dev, stream), "argmax");
    }

    // Backend<E>::quantized_matmul for E = f16 / bf16 (src/compat/mod.rs:376-378): x_dev and y_dev hold
    // elements of type `elem` (GLLMQ_ELEM_*); results are the f32 call's, rounded to nearest even.
    BackendError quantized_matmul_elem_device(const void *w_dev, size_t w_bytes, const void *x_dev, void *y_dev, QuantType t,
                                              size_t m, size_t n, size_t k, int elem, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_quantized_matmul_elem(ctx_, w_dev, w_bytes, x_dev, y_dev, static_cast<uint32_t>(t), m, n, k, elem,
                                                stream),
                    "quantized_matmul");
    }

    // The lm_head matvec of one row and Op::Argmax behind it as one call; logits_dev may be null
    // for Q6_K / Q8_0 matrices with k <= 16384 (the logits then never reach memory).
    BackendError lm_head_argmax_device(const void *w_dev, size_t w_bytes, const float *x_dev, QuantType t, size_t n, size_t k,
                                       float *logits_dev, uint32_t *token_dev, float *value_dev = nullptr,
                                       void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_lm_head_argmax(ctx_, w_dev, w_bytes, x_dev, static_cast<uint32_t>(t), n, k, logits_dev, token_dev,
                                         value_dev, stream),
                    "lm_head_argmax");
    }

    // ExpertRouteTable::from_gate_logits over device buffers (src/moe/routing.rs:100-160; graph ops
    // MoEGate + TopK, build_graph.inc.rs:2064-2071); the optional outputs may be null.
    BackendError moe_route_device(const float *logits_dev, size_t tokens, size_t experts, size_t top_k,
                                  float capacity_factor, uint32_t *route_expert_dev, float *route_weight_dev,
                                  uint32_t *route_len_dev, uint32_t *route_pos_dev = nullptr,
                                  uint32_t *expert_counts_dev = nullptr, uint32_t *overflow_dev = nullptr,
                                  void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_moe_route(ctx_, logits_dev, tokens, experts, top_k, capacity_factor, route_expert_dev,
                                    route_weight_dev, route_len_dev, route_pos_dev, expert_counts_dev, overflow_dev, stream),
                    "moe_route");
    }

    // One role of the expert weights: expert e's matrix starts at dev + e * expert_stride.
    struct ExpertWeights {
        const void *dev;
        size_t bytes;         // size of the buffer behind dev
        size_t expert_stride; // bytes between experts
    };

    // Expert FFN over a route table (ExpertRouteTable, src/moe/routing.rs:100-173).
    BackendError moe_matvec_device(ExpertWeights gate, ExpertWeights up, QuantType t_gate_up, ExpertWeights down,
                                   QuantType t_down, const float *x_dev, float *out_dev, size_t tokens, size_t hidden,
                                   size_t ffn, size_t experts, size_t top_k, const uint32_t *route_expert_dev,
                                   const float *route_weight_dev, const uint32_t *route_len_dev, bool relu_gate = false,
                                   void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_moe_matvec(ctx_, gate.dev, gate.bytes, gate.expert_stride, up.dev, up.bytes, up.expert_stride,
                                     static_cast<uint32_t>(t_gate_up), down.dev, down.bytes, down.expert_stride,
                                     static_cast<uint32_t>(t_down), x_dev, out_dev, tokens, hidden, ffn, experts, top_k,
                                     route_expert_dev, route_weight_dev, route_len_dev, relu_gate ? 1 : 0, stream),
                    "moe_matvec");
    }

    // The same for E = f32 / f16 / bf16 activations and outputs, replacing out_dev or added to it.
    BackendError moe_matvec_elem_device(ExpertWeights gate, ExpertWeights up, QuantType t_gate_up, ExpertWeights down,
                                        QuantType t_down, const void *x_dev, void *out_dev, size_t tokens, size_t hidden,
                                        size_t ffn, size_t experts, size_t top_k, const uint32_t *route_expert_dev,
                                        const float *route_weight_dev, const uint32_t *route_len_dev, int elem,
                                        bool accumulate = false, bool relu_gate = false, void *stream = nullptr) const
    {
        if (!ctx_) return init_error_;
        return make(gllmq_moe_matvec_elem(ctx_, gate.dev, gate.bytes, gate.expert_stride, up.dev, up.bytes, up.expert_stride,
                                          static_cast<uint32_t>(t_gate_up), down.dev, down.bytes, down.expert_stride,
                                          static_cast<uint32_t>(t_down), x_dev, out_dev, tokens, hidden, ffn, experts, top_k,
                                          route_expert_dev, route_weight_dev, route_len_dev, relu_gate ? 1 : 0, elem,
                                          accumulate ? GLLMQ_OUT_ACCUMULATE : 0, stream),
                    "moe_matvec");
    }

    // 1 if a chained launch since the last look ran out of its bounded wait (option
    // "chain_dependent"), 0 if none did; call after waiting for the stream.
    int chain_status() const { return ctx_ ? gllmq_chain_status(ctx_) : 0; }

    gllmq_ctx *raw() const { return ctx_; }

private:
    BackendError make(int rc, const char *what) const
    {
        if (rc == GLLMQ_OK) return BackendError{};
        std::string msg = ctx_ ? gllmq_last_error(ctx_) : "";
        if (msg.empty()) msg = std::string(what) + ": " + gllmq_status_string(rc);
        switch (rc) {
        case GLLMQ_ERR_UNIMPLEMENTED: return BackendError{ BackendError::Kind::Unimplemented, msg };
        case GLLMQ_ERR_HIP: return BackendError{ BackendError::Kind::Hip, msg };
        default: return BackendError{ BackendError::Kind::Other, msg };
        }
    }

    gllmq_ctx *ctx_ = nullptr;
    BackendError init_error_;
};

// The layers of an open GGUF file grouped by their per-layer quant-type signature, as the
// reference's graph builder groups them before it emits per-group matmul ops
// (MixedQuantPlan, src/arch/auto_graph_fragments/build_graph.inc.rs:388-470): `groups[i]` lists
// the layers of group i in ascending order, `group_of[layer]` is the layer's group (UINT32_MAX
// for a layer index without weights).  `mixed()` is false when every layer has the same signature
// (the reference's plan is None then) and both lists are empty.
struct MixedQuantPlan {
    std::vector<std::vector<size_t>> groups;
    std::vector<uint32_t> group_of;
    bool mixed() const { return !groups.empty(); }
};

inline MixedQuantPlan mixed_quant_plan(const gllmq_gguf *file)
{
    MixedQuantPlan plan;
    const size_t layers = gllmq_gguf_layer_count(file);
    std::vector<uint32_t> group_of(layers, UINT32_MAX);
    const size_t count = gllmq_gguf_mixed_quant_groups(file, group_of.data(), layers);
    if (count == 0) return plan;
    plan.groups.resize(count);
    for (size_t layer = 0; layer < layers; ++layer)
        if (group_of[layer] != UINT32_MAX) plan.groups[group_of[layer]].push_back(layer);
    plan.group_of = std::move(group_of);
    return plan;
}

} // namespace gllm

#endif
