/*
 * gllm_hip_quant: MI355X (gfx950) implementation of gllm's quantized-weight matmul path
 * behind a C ABI.  Every entry point takes plain pointers and sizes; device pointers
 * are HIP device addresses, `stream` is a hipStream_t passed as void* (NULL = the null
 * stream).  All calls are asynchronous on `stream` unless the name ends in `_host`.
 * The context's device must be the calling thread's current HIP device, and `stream` a
 * stream of that device.
 *
 * Threads and streams (Backend is Send + Sync, src/compat/mod.rs:77; the reference guards its
 * caches with a Mutex, src/compat/hip_backend.rs:22-30).  A context may be used from several
 * threads and on several streams at once: enqueues take turns on one lock, and device memory that
 * kernels use beyond their inputs and outputs ("scratch": partial sums, prepared activations,
 * intermediates) is kept per stream, so calls on different streams never share it and calls on
 * one stream are ordered by the stream.  Scratch is allocated the first time a stream needs it and
 * grows on demand; growing waits for that stream's earlier work.  Neither is possible while the
 * stream is being captured into a graph: call gllmq_reserve_* (or run the shape once) on the
 * stream before capturing, else the call returns GLLMQ_ERR_INVALID.  After that every device
 * entry point only enqueues kernels.
 *
 * Reference interfaces each entry point stands in for (paths inside putao520/gllm):
 *   Backend::quantized_matmul  src/compat/mod.rs:233-246, CPU impl src/compat/cpu_backend.rs:991-1049
 *   Backend::dequantize        src/compat/mod.rs:248-256, CPU impl src/compat/cpu_backend.rs:1051-1159
 *   Op::QuantGemm contract     src/arch/auto_graph_fragments/build_graph.inc.rs:94-123
 *   GgmlDType constants        src/loader/gguf/types.rs:57-94,152-236,443-472
 *   MoE routing / combine      src/moe/routing.rs:100-173,263-327
 *
 * Shapes follow the reference: W is n rows (outputs) of k elements stored as GGUF
 * blocks, K innermost, each row padded to whole blocks; x is [m x k], y is [m x n],
 * row-major f32.  Supported ggml dtypes: Q8_0 (8), Q4_K (12), Q5_K (13), Q6_K (14);
 * anything else returns GLLMQ_ERR_UNIMPLEMENTED, never a fallback
 * (src/compat/cpu_backend.rs:1020-1046).
 */
#ifndef GLLM_HIP_QUANT_H
#define GLLM_HIP_QUANT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GLLMQ_TYPE_Q8_0 8u
#define GLLMQ_TYPE_Q4_K 12u
#define GLLMQ_TYPE_Q5_K 13u
#define GLLMQ_TYPE_Q6_K 14u

/* Status codes.  BackendError::Unimplemented / ::Hip / ::Other of
 * src/engine/executor_types.rs:322-329 map to UNIMPLEMENTED / HIP / the rest. */
enum {
    GLLMQ_OK = 0,
    GLLMQ_ERR_UNIMPLEMENTED = 1, /* dtype or mode the library does not cover        */
    GLLMQ_ERR_BAD_SHAPE = 2,     /* sizes inconsistent with dtype/m/n/k              */
    GLLMQ_ERR_BAD_ALIGNMENT = 3, /* a device pointer misses the documented alignment */
    GLLMQ_ERR_HIP = 4,           /* a HIP runtime call failed; see gllmq_last_error  */
    GLLMQ_ERR_INVALID = 5        /* NULL context or pointer                          */
};

/* Activation handling.  The reference passes f32 activations to its CPU kernels
 * (build_graph.inc.rs:94); GLLMQ_ACT_F32_SPLIT keeps at least 22 significant bits of every
 * activation relative to the largest magnitude of its 256-element block (64-element part
 * in the GEMV kernels).  GLLMQ_ACT_BF16 rounds every activation to bf16 (nearest, ties to
 * even, as half::bf16::from_f32 does) first and then runs the same kernels: the result is
 * the exact-weight product with bf16 activations, accumulated as above. */
enum {
    GLLMQ_ACT_F32_SPLIT = 0,
    GLLMQ_ACT_BF16 = 1
};


typedef struct gllmq_ctx gllmq_ctx;

/* ---- lifetime -------------------------------------------------------------------- */
/* Loads the embedded gfx950 code object on `device` and resolves every kernel once
 * (the reference reloads its module per launch, src/compat/hip_backend.rs:211-238). */
int gllmq_init(gllmq_ctx **out_ctx, int device);
void gllmq_destroy(gllmq_ctx *ctx);
/* Message of the last failing call on this context ("" if none), copied for the calling thread:
 * valid until this thread's next gllmq_last_error. */
const char *gllmq_last_error(const gllmq_ctx *ctx);
const char *gllmq_status_string(int status);
const char *gllmq_version(void);

/* Options of a context; no counterpart in the reference.  Nothing needs setting: the defaults are
 * the measured best.  Unknown names return GLLMQ_ERR_INVALID.  Not to be changed while calls are in
 * flight on other threads.
 *
 * Supported (kept stable):
 *   "weights_cache_mib"  MiB of uploaded weights the host-slice calls keep (default 65536)
 *   "chain"              0: every entry of a batch is a launch of its own (default 1)
 *   "batch_overlap"      0: the kernels of a batch run strictly one after the other (default 1)
 *   "ffn_fused"          0: the feed-forward block as separate products (default 1)
 *   "chain_dependent"    1: an entry whose activations are the output of the entry before it stays
 *                        inside a chained launch and takes them from a mailbox in device memory as
 *                        they are stored (default 0: measured slower than a launch each, 9.0
 *                        against 8.5 us per 33 MB entry); "chain_spin_limit": looks at that mailbox
 *                        before a wave gives up (see gllmq_chain_status)
 *   "prefetch"           1: a launch on a stream of the context's own pulls the weights of each
 *                        dependent launch of a batch into the memory-side cache while the launch
 *                        before it runs (default 0: measured slower, 12.3 against 8.5 us)
 *
 * Development switches (UNSTABLE: they exist so that the test-suite and the measurements can reach
 * every kernel family through the public entry points; names and meaning may change with any
 * version, and a production caller should set none of them):
 *   kernel families on/off: "gemv_f32", "mm8", "mmf", "mm8s", "mm8s_q8_0", "mmfs", "mmfr",
 *     "moe_mm8", "moe_mm8_q6k", "moe_mm8_rows", "moe_glu", "moe_streamed", "lm_head_fused",
 *     "elem_fused", "ffn_glu_load", "ffn_streamed", "mm8s_areg", "mm8s_fold", "mm8s_split",
 *     "mm8_small_to_gemv"
 *   shape thresholds: "mm8s_min_rows", "mmfs_min_rows", "mmfr_min_rows", "chain_min_rows",
 *     "mm8_q5k_min_m", "mm8_q6k_min_m", "mm8_q8_0_min_m", "mmf_small_min_m", "mm8_ksplit",
 *     "mm8s_all", "mmfs_all" (1: that form wherever the shape fits it, also where another was timed faster)
 *   launch parameters: "mm8s_depth", "moe_depth", "moe_slices", "prefetch_wgs", "prefetch_threads",
 *     "prefetch_timeout_us", "prefetch_flags", "prefetch_announce", "prefetch_min_kib" */
int gllmq_set_option(gllmq_ctx *ctx, const char *name, long value);
/* Name of the kernel the context launched last ("" before the first launch): lets a profile be
 * matched to a call.  No counterpart in the reference. */
const char *gllmq_last_kernel_name(const gllmq_ctx *ctx);

/* Sizes the stream's scratch for a later call of that shape, so that the call itself allocates
 * nothing (needed before a stream capture).  No counterpart in the reference, whose scratch is
 * sized when the graph is compiled (src/compat/gpu_backend_macro.rs:82-87). */
int gllmq_reserve_matmul(gllmq_ctx *ctx, uint32_t ggml_dtype, size_t m, size_t n, size_t k, void *stream);
int gllmq_reserve_ffn(gllmq_ctx *ctx, uint32_t dtype_gate_up, uint32_t dtype_down, size_t m, size_t hidden,
                      size_t ffn, void *stream);
int gllmq_reserve_moe(gllmq_ctx *ctx, size_t tokens, size_t top_k, size_t hidden, size_t ffn, void *stream);

/* ---- format constants (GgmlDType::block_size / block_bytes / tensor_nbytes row rule) */
size_t gllmq_block_size(uint32_t ggml_dtype);  /* 0 if unsupported */
size_t gllmq_block_bytes(uint32_t ggml_dtype); /* 0 if unsupported */
size_t gllmq_row_bytes(uint32_t ggml_dtype, size_t k);

/* ---- Backend::dequantize ----------------------------------------------------------
 * Decodes min(n_bytes / block_bytes, n_out / block_size) whole blocks; trailing
 * partial chunks on either side are ignored (chunks_exact on both sides).
 * Alignment: none required of `blocks_dev`; `out_dev` 4 bytes. */
int gllmq_dequantize(gllmq_ctx *ctx, const void *blocks_dev, size_t n_bytes, float *out_dev,
                     size_t n_out, uint32_t ggml_dtype, void *stream);

/* ---- Op::QuantGather: quantized embedding lookup -------------------------------------
 * Replaces the graph op the reference emits when the embedding table is quantized
 * (src/arch/auto_graph_fragments/build_graph.inc.rs:203-211; table bytes
 * vocab * (hidden / block) * block_bytes, :2964-2976; scalar contract
 * (indices u32, table, output, seq_len, hidden_dim, vocab_size),
 * SPEC/MD-ARCHIVE/24-QUANT-PIPELINE-JIT.md:248-259).
 * out[i][0..hidden) = scale * dequantize(row ids[i] of the table), f32; the decoders are
 * those of gllmq_dequantize, so the values are bit-exact, and scale = 1.0f (no embedding
 * scale; the reference uses sqrt(hidden) for models that ask for one, :3009-3013) changes no
 * bit.  Table rows are gllmq_row_bytes(dtype, hidden) apart; hidden must be a multiple of 4.
 * ids live on the device and are not validated by the host: an id >= vocab produces a row
 * of NaN. */
int gllmq_quant_gather(gllmq_ctx *ctx, const void *table_dev, size_t table_bytes, uint32_t ggml_dtype,
                       size_t vocab, size_t hidden, const uint32_t *ids_dev, size_t count, float scale,
                       float *out_dev, void *stream);

/* The same with rows of another element type on the way out (Backend<E>, src/compat/mod.rs:376-378:
 * the lookup is the graph's first op and feeds activations of the model's element type): out_dev
 * holds `elem` (GLLMQ_ELEM_F32 / _F16 / _BF16) elements, each the f32 value of gllmq_quant_gather
 * rounded to nearest, ties to even; 16-bit rows are written by the lookup's own stores. */
int gllmq_quant_gather_elem(gllmq_ctx *ctx, const void *table_dev, size_t table_bytes, uint32_t ggml_dtype,
                            size_t vocab, size_t hidden, const uint32_t *ids_dev, size_t count, float scale,
                            void *out_dev, int elem, void *stream);

/* ---- Dense feed-forward block: gate/up projections, SwiGLU, down projection -------------
 * Replaces the op sequence the reference emits per layer (QuantGemm gate_proj, QuantGemm
 * up_proj, Op::SwiGlu, QuantGemm down_proj: src/arch/auto_graph_fragments/
 * build_graph.inc.rs:1957-1995; formula down(silu(gate x) * (up x)), SPEC 04-OPERATORS.md:114):
 *   out[m x hidden] = ( act(x . Wgate^T) * (x . Wup^T) ) . Wdown^T,   act = SiLU
 * (relu_gate != 0: SiLU behind a ReLU).  Wgate and Wup are [ffn x hidden] of dtype_gate_up,
 * each of gate_up_bytes_each bytes; Wdown is [hidden x ffn] of dtype_down; x and out are f32.
 * Q4_K / Q5_K gate and up with up to 8 rows run as ONE launch of the int8 matrix-core kernel
 * with the activation in its epilogue (a workgroup runs the gate tile and the up tile of a
 * row range back to back); other shapes run the two products (one matmul when the up rows
 * follow the gate rows in memory), an activation kernel and the down projection, each with
 * the kernels gllmq_quantized_matmul would pick.  Intermediates live in the stream's scratch. */
int gllmq_ffn_swiglu(gllmq_ctx *ctx, const void *gate_dev, const void *up_dev, size_t gate_up_bytes_each,
                     uint32_t dtype_gate_up, const void *down_dev, size_t down_bytes, uint32_t dtype_down,
                     const float *x_dev, float *out_dev, size_t m, size_t hidden, size_t ffn, int relu_gate,
                     void *stream);

/* The same over activations and outputs of element type `elem` (Backend<E>, src/compat/mod.rs:376-378),
 * and, with GLLMQ_OUT_ACCUMULATE in `flags`, added to what out_dev holds instead of replacing it:
 * the Op::Add that puts a shared expert's feed-forward block on top of the routed experts' sum, and
 * the residual add behind the block (build_graph.inc.rs:2132-2170).  16-bit activations widen
 * exactly; the block runs in f32 as gllmq_ffn_swiglu does; out = round(result) or
 * out = round(widen(out) + result), one rounding to nearest, ties to even (f32: none beyond the
 * addition's).  Bit for bit: the result of gllmq_ffn_swiglu on the widened activations, added and
 * rounded.  The conversions are small launches of their own around the block's kernels. */
#define GLLMQ_OUT_ACCUMULATE 1
int gllmq_ffn_swiglu_elem(gllmq_ctx *ctx, const void *gate_dev, const void *up_dev, size_t gate_up_bytes_each,
                          uint32_t dtype_gate_up, const void *down_dev, size_t down_bytes, uint32_t dtype_down,
                          const void *x_dev, void *out_dev, size_t m, size_t hidden, size_t ffn, int relu_gate,
                          int elem, int flags, void *stream);

/* ---- Op::Argmax: greedy token choice behind the lm_head matmul -----------------------
 * Replaces the graph op of src/arch/auto_graph_fragments/build_graph.inc.rs:2661 with the
 * semantics of argmax_token (src/engine/executor_step.rs:48-55; its unit tests :2191-2325):
 * token_dev[r] = index of the largest entry of row r that is not NaN; of equal maxima the
 * LAST one wins; GLLMQ_ARGMAX_NONE when the row is empty or all NaN (the reference's None).
 * logits_dev is [rows][ld] f32 with n <= ld entries used per row; value_dev (may be NULL)
 * receives the winning logit (NaN for no token).  The keys between the two launches live in the
 * stream's scratch. */
#define GLLMQ_ARGMAX_NONE 0xFFFFFFFFu
int gllmq_argmax(gllmq_ctx *ctx, const float *logits_dev, size_t rows, size_t n, size_t ld,
                 uint32_t *token_dev, float *value_dev, void *stream);

/* ---- Backend<E>::quantized_matmul for E = f16 and bf16 -------------------------------
 * The reference's backend trait is generic over the element type of activations and outputs
 * (Backend<E: Element>, f32 / half::f16 / half::bf16: src/compat/mod.rs:376-378;
 * quantized_matmul takes input: &[E] and output: &mut [E], src/compat/mod.rs:233-246).
 * x_dev holds m x k and y_dev m x n elements of type `elem`; 16-bit activations widen exactly,
 * the arithmetic is that of gllmq_quantized_matmul, and a result is rounded to the nearest
 * element, ties to even (what E::from_f32 does; NaN stays NaN, f16 overflows to infinity): y is
 * bit for bit the rounded result of the f32 call on the widened activations.  The streamed
 * kernels, the GEMV (rows that are aligned vectors, k <= 16384) and the GEMM convert in their own
 * loads and stores; other shapes take a widening and a rounding launch around the f32 kernels,
 * through scratch of the stream (gllmq_reserve_matmul_elem before capturing such a shape).
 * Both pointers 4-byte aligned. */
#define GLLMQ_ELEM_F32 0
#define GLLMQ_ELEM_F16 1
#define GLLMQ_ELEM_BF16 2
int gllmq_quantized_matmul_elem(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const void *x_dev, void *y_dev,
                                uint32_t ggml_dtype, size_t m, size_t n, size_t k, int elem, void *stream);
int gllmq_reserve_matmul_elem(gllmq_ctx *ctx, uint32_t ggml_dtype, size_t m, size_t n, size_t k, int elem, void *stream);

/* ---- lm_head matvec and Op::Argmax as one call ---------------------------------------
 * The tail of a decode step: the lm_head MatMul of one activation row (reached through
 * Backend::quantized_matmul, src/compat/cpu_backend.rs:991-1049) followed by Op::Argmax
 * (build_graph.inc.rs:2661).  w_dev is [n x k] of ggml_dtype, x_dev k f32; token_dev and
 * value_dev as in gllmq_argmax (one row).  logits_dev (n f32) receives the logits; it may be
 * NULL when only the token is wanted and the matrix is Q6_K or Q8_0 with k <= 16384: there
 * every workgroup of the matvec leaves its best candidate behind and the one that finishes last
 * picks among them (one launch), so the logits are neither written nor read again.  Other matrices run
 * gllmq_quantized_matmul and gllmq_argmax one after the other and need logits_dev, and so do
 * shapes with a logits buffer for which gllmq_quantized_matmul has a faster kernel than that
 * matvec (Q8_0 rows of whole 256-element groups, a few long Q6_K rows).  With logits_dev the
 * logits and the token are those of the two calls made separately, bit for bit; without it the
 * token is the choice among that matvec's own logits, which agree with the other kernels' to the
 * matmul's tolerance. */
int gllmq_lm_head_argmax(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const float *x_dev, uint32_t ggml_dtype,
                         size_t n, size_t k, float *logits_dev, uint32_t *token_dev, float *value_dev, void *stream);

/* ---- Backend::quantized_matmul ----------------------------------------------------
 * y[m x n] = x[m x k] . W[n x k]^T.  w_bytes must be at least n * gllmq_row_bytes(dtype,k).
 * Alignment: w_dev 16 bytes for Q4_K/Q5_K, 2 bytes for Q6_K/Q8_0; x_dev 16, y_dev 4.
 * Q4_K runs on the int8 matrix cores: activations become three signed base-256 digits of a
 * per-block fixed-point value, digit products accumulate exactly in i32, scales and the
 * final sum are f32; one pass over the weights serves up to 8 activation rows.  Q5_K with 2
 * or more rows, Q6_K and Q8_0 with 3 or more run the same scheme (Q8_0: one matrix-core step
 * per 32-element block, its f16 scale applied in f32).  More than 8 rows run a GEMM on the
 * f16 matrix cores, 64 rows per pass: weights as the exact integers sc*q in f16 (Q6_K: q-32,
 * Q8_0: q, their scales applied per 16 or 32 elements in f32), activations as two f16 terms
 * (22 significant bits) of a per-block scaled value, f32 accumulation; its activation images
 * and the partial sums of its K split live in the stream's scratch.  The GEMM also takes 3..8 rows when the rows are so
 * long that the prepared activations do not fit the LDS of one 8-row pass (K above about
 * 4096..12288, by format and rows).  Q5_K with one row, Q6_K and Q8_0 with one or two, and
 * Q8_0 rows shorter than 256 elements run integer-dot GEMV kernels, two activation rows per
 * pass; one Q5_K or Q6_K row of 40 blocks and more over at most 4096 weight rows takes the
 * matrix-core kernel.  With so few weight rows that their 32-row tiles cover at most half of
 * the CUs, the matrix-core kernels of up to 8 rows split K across the workgroups of one launch
 * (the last workgroup of a tile adds the slice sums in slice order); slice sums and arrival
 * counters live in the stream's scratch too. */
int gllmq_quantized_matmul(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const float *x_dev,
                           float *y_dev, uint32_t ggml_dtype, size_t m, size_t n, size_t k,
                           void *stream);

/* Same, with the activation mode chosen by the caller. */
int gllmq_quantized_matmul_ex(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes,
                              const float *x_dev, float *y_dev, uint32_t ggml_dtype, size_t m,
                              size_t n, size_t k, int act_mode, void *stream);

/* ---- the quantized matmul for callers that cannot allocate ---------------------------------
 * No counterpart in the reference.  For callers that cannot call hipMalloc: code under stream
 * capture, tight serving loops, harnesses that forbid allocation.  Same arguments, same kernels
 * and bit-identical results as gllmq_quantized_matmul, but the scratch (arrival counters and slice
 * sums of the K split, activation images and partial sums of the GEMM) is one array of
 * GLLMQ_NOALLOC_SCRATCH_BYTES in device memory whose address gllmq_init looks up for the context's
 * device (that lookup is what places the array there, so init fails if it cannot; every GPU the
 * library runs on holds its own copy until the process ends); the call itself allocates and frees
 * nothing and may be the first call on a fresh context, also under stream capture.  A shape whose scratch does not fit (the GEMM's: about 72 KiB per 256
 * elements of K for up to 64 rows plus ksplit * min(m, 64) * n * 4 bytes of partial sums, in
 * 27.9 MiB) returns GLLMQ_ERR_BAD_SHAPE with the two sizes in gllmq_last_error; every baseline
 * shape up to 64 rows fits.  All calls on one GPU share that GPU's array, whatever their context
 * or stream: calls that overlap in time on one GPU race, so keep them on one stream or order them
 * yourself.  The context's device must be the calling thread's current device (checked on every
 * call). */
#define GLLMQ_NOALLOC_SCRATCH_BYTES (32u << 20)
int gllmq_quantized_matmul_noalloc(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const float *x_dev,
                                   float *y_dev, uint32_t ggml_dtype, size_t m, size_t n, size_t k,
                                   void *stream);

/* A list of matmuls enqueued on one stream from one call (the QuantGemm ops of one decode layer
 * = QKV, O, gate/up, down: build_graph.inc.rs:1960-1999).  The entries are taken to be independent
 * of each other (no entry reads what another writes): their kernels may overlap in time on the
 * device, and consecutive one- or two-row Q4_K / Q5_K entries of one K <= 4096 run as ONE launch
 * whose loaders go straight on from one matrix to the next (up to 32 entries per launch), which
 * saves the gaps between kernels and keeps the weight stream going.  An entry that does depend on the entries before it carries
 * GLLMQ_DESC_AFTER_PREVIOUS in `flags`: it starts after they have finished.  The batch as a whole
 * is ordered like any other call: it starts after the stream's earlier work and later work
 * starts after all of it.  GLLMQ_DESC_ELEM_F16 / _BF16: x_dev and y_dev of the entry hold elements
 * of that type (as for gllmq_quantized_matmul_elem; such an entry is a launch of its own). */
#define GLLMQ_DESC_AFTER_PREVIOUS 1u
#define GLLMQ_DESC_ELEM_F16 0x100u
#define GLLMQ_DESC_ELEM_BF16 0x200u
typedef struct gllmq_matmul_desc {
    const void *w_dev;
    size_t w_bytes;
    const float *x_dev;
    float *y_dev;
    uint32_t ggml_dtype;
    uint32_t flags; /* 0 or GLLMQ_DESC_* bits */
    size_t m, n, k;
} gllmq_matmul_desc;

int gllmq_quantized_matmul_batch(gllmq_ctx *ctx, const gllmq_matmul_desc *descs, size_t count,
                                 void *stream);

/* With option "chain_dependent" an entry whose activations are the output of the entry before it
 * stays inside the chained launch and waits there for those outputs, a bounded number of looks
 * (option "chain_spin_limit"); a wave whose wait runs out goes on with what it has, so the launch
 * always ends, and raises a word in host-visible memory.  That word is looked at by the NEXT
 * gllmq_quantized_matmul_batch call on the context, which fails with GLLMQ_ERR_HIP once (the
 * outputs of the launch that timed out are invalid), and by this function: after the caller has
 * waited for the stream, 1 if a chained launch since the last look timed out (and the word is set
 * back, so the next batch call reports nothing), 0 if none did.  No counterpart in the reference,
 * whose decode step has no waits of its own. */
int gllmq_chain_status(gllmq_ctx *ctx);

/* ---- MoE router: gate logits -> route table ------------------------------------------
 * Replaces the graph ops MoEGate + TopK (src/arch/auto_graph_fragments/build_graph.inc.rs:2064-2071)
 * and their host mirror ExpertRouteTable::from_gate_logits (src/moe/routing.rs:100-160) over
 * topk_with_weights / softmax (src/moe/routing.rs:263-302).  Per token: p = softmax(logits) (sum
 * in expert order; all p = 1/experts when the sum is not positive), the min(top_k, experts)
 * largest p in descending order with the lower index first among equals (a stable sort),
 * weights divided by their sum.  Then, tokens in order, a choice is kept while its expert holds
 * fewer than capacity = ceil(capacity_factor * tokens / experts) tokens (f32 arithmetic, clamped
 * to [0, 1e9], src/moe/routing.rs:53-61; the reference's default factor is 1.25, :40-49); a
 * token whose choices are all full goes to the least loaded expert (the first of equals) with
 * weight 1.0.  logits_dev is [tokens x experts] f32; the outputs are the [tokens x top_k] /
 * [tokens] arrays gllmq_moe_matvec takes (entries past route_len[t] are written as 0);
 * route_pos_dev (the token's position in its expert's list), expert_counts_dev [experts] and
 * overflow_dev [1] (choices dropped) may be NULL.  exp() is the device's: a weight may differ
 * from a libm-based host by an ulp or two, and two experts whose probabilities collide within
 * that may swap places.
 * Limits of this build: experts <= 4096, top_k <= 64.  Up to 64 tokens this is one launch. */
int gllmq_moe_route(gllmq_ctx *ctx, const float *logits_dev, size_t tokens, size_t experts, size_t top_k,
                    float capacity_factor, uint32_t *route_expert_dev, float *route_weight_dev,
                    uint32_t *route_len_dev, uint32_t *route_pos_dev, uint32_t *expert_counts_dev,
                    uint32_t *overflow_dev, void *stream);

/* ---- MoE expert matvec (ExpertRouteTable grouping, src/moe/routing.rs:163-173) -----
 * out[t] = sum_i weight[t][i] * down_e( silu(gate_e x_t) * (up_e x_t) ), e = expert[t][i],
 * summed in route order i = 0 .. route_len[t]-1 (src/moe/routing.rs:307-327); a token with
 * no route gets zeros.  Only routed (token, expert) pairs are computed (the reference graph
 * runs every expert on every token and masks, build_graph.inc.rs:2076-2123).  Q4_K, Q5_K and
 * Q6_K rows of at most 4096 elements run on the int8 matrix cores, all tokens of an expert
 * (eight per pass) against one read of its weights, Q4_K / Q5_K gate and up with the activation
 * in the same launch; other shapes run the integer-dot GEMV, two tokens per pass.
 * Expert e's gate rows ([ffn x hidden] blocks of dtype_gate_up) start at gate_dev +
 * e * gate_expert_stride, its up rows at up_dev + e * up_expert_stride, its down rows
 * ([hidden x ffn] of dtype_down) at down_dev + e * down_expert_stride; *_bytes are the sizes of
 * the three buffers, and every expert's matrix must lie inside its buffer.  This covers both
 * layouts in use: the reference's, one stride over an expert's three matrices (gate, up, down
 * back to back, build_graph.inc.rs:2080-2125: the three pointers are offsets into one buffer and
 * the three strides are equal), and GGUF's, one stacked tensor per role (stride = one matrix).
 * route_* are [tokens x top_k] device arrays, route_len[t] entries valid per token; entries
 * past route_len[t] are ignored and an expert index >= experts routes nowhere (device data is
 * not validated on the host).  relu_gate != 0 applies max(g,0) before silu.
 * Limits of this build: tokens*top_k <= 16384, experts <= 4096, hidden and ffn <= 16384
 * and multiples of 4 (else GLLMQ_ERR_UNIMPLEMENTED / BAD_SHAPE).  x_dev 16-byte aligned;
 * weights and strides aligned as for gllmq_quantized_matmul.
 * Intermediate buffers live in the stream's scratch. */
int gllmq_moe_matvec(gllmq_ctx *ctx, const void *gate_dev, size_t gate_bytes, size_t gate_expert_stride,
                     const void *up_dev, size_t up_bytes, size_t up_expert_stride, uint32_t dtype_gate_up,
                     const void *down_dev, size_t down_bytes, size_t down_expert_stride, uint32_t dtype_down,
                     const float *x_dev, float *out_dev, size_t tokens, size_t hidden, size_t ffn, size_t experts,
                     size_t top_k, const uint32_t *route_expert_dev, const float *route_weight_dev,
                     const uint32_t *route_len_dev, int relu_gate, void *stream);

/* gllmq_moe_matvec over activations and outputs of element type `elem`, and with
 * GLLMQ_OUT_ACCUMULATE added to out_dev (see gllmq_ffn_swiglu_elem: same rules, same rounding). */
int gllmq_moe_matvec_elem(gllmq_ctx *ctx, const void *gate_dev, size_t gate_bytes, size_t gate_expert_stride,
                          const void *up_dev, size_t up_bytes, size_t up_expert_stride, uint32_t dtype_gate_up,
                          const void *down_dev, size_t down_bytes, size_t down_expert_stride, uint32_t dtype_down,
                          const void *x_dev, void *out_dev, size_t tokens, size_t hidden, size_t ffn, size_t experts,
                          size_t top_k, const uint32_t *route_expert_dev, const float *route_weight_dev,
                          const uint32_t *route_len_dev, int relu_gate, int elem, int flags, void *stream);

/* ---- GGUF reader and tensor upload ---------------------------------------------------
 * The file side of the path: what the reference's loader accepts and rejects
 * (src/loader/gguf/reader.rs:38-187): magic "GGUF", version 3 only, key/value metadata,
 * tensor infos, `general.alignment` (default 32, 0 is an error), tensor data from the aligned
 * end of the infos, every tensor inside the file, no duplicate names; a tensor's bytes are
 * ceil(ne0 / block) * block_bytes * ne1 * ... for all 36 dtype ids of
 * src/loader/gguf/types.rs:57-94,152-236,443-472.  The file is mapped read-only and the
 * tensor data is uploaded straight from the mapping.  Host only: needs no GPU except
 * gllmq_gguf_upload.  Strings handed out are NOT zero-terminated views into the file
 * (length returned beside them) except tensor names. */
typedef struct gllmq_gguf gllmq_gguf;

enum {
    GLLMQ_GGUF_OK = 0,
    GLLMQ_GGUF_ERR_IO = 1,       /* GgufError::Io */
    GLLMQ_GGUF_ERR_MAGIC = 2,    /* GgufError::InvalidMagic */
    GLLMQ_GGUF_ERR_VERSION = 3,  /* GgufError::UnsupportedVersion */
    GLLMQ_GGUF_ERR_PARSE = 4,    /* GgufError::ParseError (truncated file, overflow, duplicate name, ...) */
    GLLMQ_GGUF_ERR_METADATA = 5, /* GgufError::InvalidMetadata */
    GLLMQ_GGUF_ERR_BOUNDS = 6,   /* GgufError::TensorOutOfBounds */
    GLLMQ_GGUF_ERR_DTYPE = 7,    /* a ggml dtype id outside the table */
    GLLMQ_GGUF_ERR_UTF8 = 8      /* GgufError::Utf8: a key, string value or tensor name that is not UTF-8 */
};

typedef struct gllmq_gguf_tensor {
    const char *name;     /* zero-terminated, owned by the reader */
    uint32_t ggml_dtype;
    uint32_t n_dims;      /* 0..4 */
    uint64_t shape[4];    /* outermost first, as the reference hands shapes to its consumers
                             (reader.rs:593-598): a [n x k] weight reads {n, k} */
    uint64_t ne[4];       /* as stored: ne[0] innermost */
    size_t offset;        /* absolute position in the file */
    size_t nbytes;
} gllmq_gguf_tensor;

int gllmq_gguf_open(const char *path, gllmq_gguf **out, char *err, size_t err_len);
/* the same over an image in memory, which must outlive the reader */
int gllmq_gguf_parse(const void *bytes, size_t len, gllmq_gguf **out, char *err, size_t err_len);
void gllmq_gguf_close(gllmq_gguf *g);
uint32_t gllmq_gguf_version(const gllmq_gguf *g);
size_t gllmq_gguf_tensor_count(const gllmq_gguf *g);
size_t gllmq_gguf_kv_count(const gllmq_gguf *g);
size_t gllmq_gguf_alignment(const gllmq_gguf *g);
size_t gllmq_gguf_data_offset(const gllmq_gguf *g);
int gllmq_gguf_tensor_at(const gllmq_gguf *g, size_t index, gllmq_gguf_tensor *out);
long gllmq_gguf_find_tensor(const gllmq_gguf *g, const char *name); /* -1: no such tensor */
const void *gllmq_gguf_tensor_data(const gllmq_gguf *g, size_t index);
/* The per-layer weights `blk.{layer}.{projection}.weight` (attn_q, attn_k, attn_v, attn_output,
 * ffn_gate, ffn_up, ffn_down, ...) as a table: what a host walks to call the kernels with each
 * matrix's own format, `*_K_M` files mixing Q4_K / Q5_K with Q6_K from layer to layer.
 * gllmq_gguf_layer_count: highest layer index + 1 (0: no such tensors);
 * gllmq_gguf_layer_tensors: number of weights of `layer`, their tensor indices in projection-name
 * order into indices[0 .. capacity); gllmq_gguf_layer_tensor: index of one of them or -1.
 * gllmq_gguf_mixed_quant_groups: the reference's grouping of layers by dtype signature (the sorted
 * (projection, dtype) pairs of a layer; src/arch/auto_graph_fragments/build_graph.inc.rs:388-470):
 * returns 0 when every layer has the same signature (the reference's plan is None then), else the
 * number of groups, numbered in signature order; group_of[layer] (layer < capacity) receives the
 * layer's group, UINT32_MAX for a layer index without weights. */
size_t gllmq_gguf_layer_count(const gllmq_gguf *g);
size_t gllmq_gguf_layer_tensors(const gllmq_gguf *g, size_t layer, size_t *indices, size_t capacity);
long gllmq_gguf_layer_tensor(const gllmq_gguf *g, size_t layer, const char *projection);
size_t gllmq_gguf_mixed_quant_groups(const gllmq_gguf *g, uint32_t *group_of, size_t capacity);
/* metadata: the GgufValueType id (0..12) of a key or -1; the getters return 1 when the key
 * exists and converts (gllmq_gguf_meta_u64 like GgufValue::as_u64: unsigned kinds, and signed
 * kinds that are not negative), else 0 */
int gllmq_gguf_meta_type(const gllmq_gguf *g, const char *key);
int gllmq_gguf_meta_u64(const gllmq_gguf *g, const char *key, uint64_t *out);
int gllmq_gguf_meta_i64(const gllmq_gguf *g, const char *key, int64_t *out);
int gllmq_gguf_meta_f64(const gllmq_gguf *g, const char *key, double *out);
int gllmq_gguf_meta_bool(const gllmq_gguf *g, const char *key, int *out);
const char *gllmq_gguf_meta_str(const gllmq_gguf *g, const char *key, size_t *len);
int gllmq_gguf_meta_array(const gllmq_gguf *g, const char *key, uint32_t *item_type, uint64_t *count);
const char *gllmq_gguf_meta_array_str(const gllmq_gguf *g, const char *key, uint64_t index, size_t *len);
/* tensor `index` into device memory (dst_bytes >= its nbytes), as the file stores it: the
 * layout gllmq_quantized_matmul, gllmq_quant_gather and gllmq_ffn_swiglu take */
int gllmq_gguf_upload(gllmq_ctx *ctx, const gllmq_gguf *g, size_t index, void *dst_dev, size_t dst_bytes,
                      void *stream);

/* ---- host-slice forms: the literal signatures of the trait (upload, run, download, synchronise)
 * The weight slice (blocks / table / w) is uploaded the first time it is seen and kept on the
 * device, keyed by its address and length, as the reference keeps its uploaded weight blob
 * (src/compat/hip_backend.rs:141-156): later calls with the same slice copy only activations and
 * results.  Weights behind a cached slice must not change; gllmq_weights_forget(ctx, ptr) drops
 * one slice (NULL: all) before its memory is reused.  gllmq_weight_uploads counts the
 * host-to-device weight copies a context has made. */
void gllmq_weights_forget(gllmq_ctx *ctx, const void *host_ptr);
uint64_t gllmq_weight_uploads(const gllmq_ctx *ctx);
int gllmq_dequantize_host(gllmq_ctx *ctx, const void *blocks, size_t n_bytes, float *out,
                          size_t n_out, uint32_t ggml_dtype);
int gllmq_quant_gather_host(gllmq_ctx *ctx, const void *table, size_t table_bytes, uint32_t ggml_dtype,
                            size_t vocab, size_t hidden, const uint32_t *ids, size_t count, float scale, float *out);
int gllmq_quantized_matmul_host(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x,
                                float *y, uint32_t ggml_dtype, size_t m, size_t n, size_t k);

#ifdef __cplusplus
}
#endif
#endif
