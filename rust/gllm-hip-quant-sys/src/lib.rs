//! Raw bindings to `libgllm_hip_quant.so` (include/gllm_hip_quant.h) and the safe wrapper that
//! plugs into gllm's `Backend` trait for the quantized-weight matmul path.
//!
//! Replaces the `Unimplemented` defaults of `Backend::quantized_matmul` / `Backend::dequantize`
//! (src/compat/mod.rs:233-256) for the HIP backend (src/compat/hip_backend.rs).
#![allow(non_camel_case_types)]

use std::ffi::{c_char, c_int, c_void, CStr};

#[repr(C)]
pub struct gllmq_ctx {
    _private: [u8; 0],
}

#[repr(C)]
#[derive(Clone, Copy)]
pub struct gllmq_matmul_desc {
    pub w_dev: *const c_void,
    pub w_bytes: usize,
    pub x_dev: *const f32,
    pub y_dev: *mut f32,
    pub ggml_dtype: u32,
    pub flags: u32, // GLLMQ_DESC_AFTER_PREVIOUS (1): the entry depends on the entries before it; GLLMQ_DESC_ELEM_F16 (0x100) / _BF16 (0x200): x and y hold such elements
    pub m: usize,
    pub n: usize,
    pub k: usize,
}

pub const GLLMQ_OK: c_int = 0;
pub const GLLMQ_ERR_UNIMPLEMENTED: c_int = 1;
pub const GLLMQ_ERR_BAD_SHAPE: c_int = 2;
pub const GLLMQ_ERR_BAD_ALIGNMENT: c_int = 3;
pub const GLLMQ_ERR_HIP: c_int = 4;
pub const GLLMQ_ERR_INVALID: c_int = 5;
pub const GLLMQ_ACT_F32_SPLIT: c_int = 0;
pub const GLLMQ_ACT_BF16: c_int = 1;

/// `flags` of the `_elem` block entry points: add to the output instead of replacing it.
pub const GLLMQ_OUT_ACCUMULATE: c_int = 1;

extern "C" {
    pub fn gllmq_init(out_ctx: *mut *mut gllmq_ctx, device: c_int) -> c_int;
    pub fn gllmq_destroy(ctx: *mut gllmq_ctx);
    pub fn gllmq_last_error(ctx: *const gllmq_ctx) -> *const c_char;
    pub fn gllmq_status_string(status: c_int) -> *const c_char;
    pub fn gllmq_version() -> *const c_char;
    pub fn gllmq_block_size(ggml_dtype: u32) -> usize;
    pub fn gllmq_block_bytes(ggml_dtype: u32) -> usize;
    pub fn gllmq_row_bytes(ggml_dtype: u32, k: usize) -> usize;
    pub fn gllmq_dequantize(ctx: *mut gllmq_ctx, blocks_dev: *const c_void, n_bytes: usize, out_dev: *mut f32,
                            n_out: usize, ggml_dtype: u32, stream: *mut c_void) -> c_int;
    pub fn gllmq_quantized_matmul(ctx: *mut gllmq_ctx, w_dev: *const c_void, w_bytes: usize, x_dev: *const f32,
                                  y_dev: *mut f32, ggml_dtype: u32, m: usize, n: usize, k: usize,
                                  stream: *mut c_void) -> c_int;
    pub fn gllmq_quantized_matmul_ex(ctx: *mut gllmq_ctx, w_dev: *const c_void, w_bytes: usize, x_dev: *const f32,
                                     y_dev: *mut f32, ggml_dtype: u32, m: usize, n: usize, k: usize,
                                     act_mode: c_int, stream: *mut c_void) -> c_int;
    pub fn gllmq_quantized_matmul_batch(ctx: *mut gllmq_ctx, descs: *const gllmq_matmul_desc, count: usize,
                                        stream: *mut c_void) -> c_int;
    pub fn gllmq_chain_status(ctx: *mut gllmq_ctx) -> c_int;
    pub fn gllmq_quant_gather_elem(ctx: *mut gllmq_ctx, table_dev: *const c_void, table_bytes: usize, ggml_dtype: u32,
                                   vocab: usize, hidden: usize, ids_dev: *const u32, count: usize, scale: f32,
                                   out_dev: *mut c_void, elem: c_int, stream: *mut c_void) -> c_int;
    pub fn gllmq_ffn_swiglu_elem(ctx: *mut gllmq_ctx, gate_dev: *const c_void, up_dev: *const c_void,
                                 gate_up_bytes_each: usize, dtype_gate_up: u32, down_dev: *const c_void, down_bytes: usize,
                                 dtype_down: u32, x_dev: *const c_void, out_dev: *mut c_void, m: usize, hidden: usize,
                                 ffn: usize, relu_gate: c_int, elem: c_int, flags: c_int, stream: *mut c_void) -> c_int;
    pub fn gllmq_moe_matvec_elem(ctx: *mut gllmq_ctx, gate_dev: *const c_void, gate_bytes: usize, gate_expert_stride: usize,
                                 up_dev: *const c_void, up_bytes: usize, up_expert_stride: usize, dtype_gate_up: u32,
                                 down_dev: *const c_void, down_bytes: usize, down_expert_stride: usize, dtype_down: u32,
                                 x_dev: *const c_void, out_dev: *mut c_void, tokens: usize, hidden: usize, ffn: usize,
                                 experts: usize, top_k: usize, route_expert_dev: *const u32, route_weight_dev: *const f32,
                                 route_len_dev: *const u32, relu_gate: c_int, elem: c_int, flags: c_int,
                                 stream: *mut c_void) -> c_int;
    pub fn gllmq_moe_route(ctx: *mut gllmq_ctx, logits_dev: *const f32, tokens: usize, experts: usize, top_k: usize,
                           capacity_factor: f32, route_expert_dev: *mut u32, route_weight_dev: *mut f32,
                           route_len_dev: *mut u32, route_pos_dev: *mut u32, expert_counts_dev: *mut u32,
                           overflow_dev: *mut u32, stream: *mut c_void) -> c_int;
    pub fn gllmq_moe_matvec(ctx: *mut gllmq_ctx, gate_dev: *const c_void, gate_bytes: usize, gate_expert_stride: usize,
                            up_dev: *const c_void, up_bytes: usize, up_expert_stride: usize, dtype_gate_up: u32,
                            down_dev: *const c_void, down_bytes: usize, down_expert_stride: usize, dtype_down: u32,
                            x_dev: *const f32, out_dev: *mut f32,
                            tokens: usize, hidden: usize, ffn: usize, experts: usize, top_k: usize,
                            route_expert_dev: *const u32, route_weight_dev: *const f32,
                            route_len_dev: *const u32, relu_gate: c_int, stream: *mut c_void) -> c_int;
    pub fn gllmq_set_option(ctx: *mut gllmq_ctx, name: *const c_char, value: std::os::raw::c_long) -> c_int;
    pub fn gllmq_last_kernel_name(ctx: *const gllmq_ctx) -> *const c_char;
    pub fn gllmq_reserve_matmul(ctx: *mut gllmq_ctx, ggml_dtype: u32, m: usize, n: usize, k: usize,
                                stream: *mut c_void) -> c_int;
    pub fn gllmq_reserve_ffn(ctx: *mut gllmq_ctx, dtype_gate_up: u32, dtype_down: u32, m: usize, hidden: usize,
                             ffn: usize, stream: *mut c_void) -> c_int;
    pub fn gllmq_reserve_moe(ctx: *mut gllmq_ctx, tokens: usize, top_k: usize, hidden: usize, ffn: usize,
                             stream: *mut c_void) -> c_int;
    pub fn gllmq_weights_forget(ctx: *mut gllmq_ctx, host_ptr: *const c_void);
    pub fn gllmq_weight_uploads(ctx: *const gllmq_ctx) -> u64;
    pub fn gllmq_ffn_swiglu(ctx: *mut gllmq_ctx, gate_dev: *const c_void, up_dev: *const c_void,
                            gate_up_bytes_each: usize, dtype_gate_up: u32, down_dev: *const c_void, down_bytes: usize,
                            dtype_down: u32, x_dev: *const f32, out_dev: *mut f32, m: usize, hidden: usize,
                            ffn: usize, relu_gate: c_int, stream: *mut c_void) -> c_int;
    pub fn gllmq_argmax(ctx: *mut gllmq_ctx, logits_dev: *const f32, rows: usize, n: usize, ld: usize,
                        token_dev: *mut u32, value_dev: *mut f32, stream: *mut c_void) -> c_int;
    pub fn gllmq_quantized_matmul_elem(ctx: *mut gllmq_ctx, w_dev: *const c_void, w_bytes: usize, x_dev: *const c_void,
                                       y_dev: *mut c_void, ggml_dtype: u32, m: usize, n: usize, k: usize, elem: c_int,
                                       stream: *mut c_void) -> c_int;
    pub fn gllmq_reserve_matmul_elem(ctx: *mut gllmq_ctx, ggml_dtype: u32, m: usize, n: usize, k: usize, elem: c_int,
                                     stream: *mut c_void) -> c_int;
    pub fn gllmq_lm_head_argmax(ctx: *mut gllmq_ctx, w_dev: *const c_void, w_bytes: usize, x_dev: *const f32,
                                ggml_dtype: u32, n: usize, k: usize, logits_dev: *mut f32, token_dev: *mut u32,
                                value_dev: *mut f32, stream: *mut c_void) -> c_int;
    pub fn gllmq_quant_gather(ctx: *mut gllmq_ctx, table_dev: *const c_void, table_bytes: usize, ggml_dtype: u32,
                              vocab: usize, hidden: usize, ids_dev: *const u32, count: usize, scale: f32,
                              out_dev: *mut f32, stream: *mut c_void) -> c_int;
    pub fn gllmq_quant_gather_host(ctx: *mut gllmq_ctx, table: *const c_void, table_bytes: usize, ggml_dtype: u32,
                                   vocab: usize, hidden: usize, ids: *const u32, count: usize, scale: f32,
                                   out: *mut f32) -> c_int;
    // GGUF reader (src/loader/gguf/reader.rs:38-187) and upload; the reader is an opaque handle
    pub fn gllmq_gguf_open(path: *const c_char, out: *mut *mut c_void, err: *mut c_char, err_len: usize) -> c_int;
    pub fn gllmq_gguf_close(g: *mut c_void);
    pub fn gllmq_gguf_tensor_count(g: *const c_void) -> usize;
    pub fn gllmq_gguf_find_tensor(g: *const c_void, name: *const c_char) -> std::os::raw::c_long;
    pub fn gllmq_gguf_tensor_data(g: *const c_void, index: usize) -> *const c_void;
    pub fn gllmq_gguf_upload(ctx: *mut gllmq_ctx, g: *const c_void, index: usize, dst_dev: *mut c_void,
                             dst_bytes: usize, stream: *mut c_void) -> c_int;
    // per-layer weight table and the grouping of layers by dtype signature
    // (src/arch/auto_graph_fragments/build_graph.inc.rs:388-470)
    pub fn gllmq_gguf_layer_count(g: *const c_void) -> usize;
    pub fn gllmq_gguf_layer_tensors(g: *const c_void, layer: usize, indices: *mut usize, capacity: usize) -> usize;
    pub fn gllmq_gguf_layer_tensor(g: *const c_void, layer: usize, projection: *const c_char) -> std::os::raw::c_long;
    pub fn gllmq_gguf_mixed_quant_groups(g: *const c_void, group_of: *mut u32, capacity: usize) -> usize;
    pub fn gllmq_dequantize_host(ctx: *mut gllmq_ctx, blocks: *const c_void, n_bytes: usize, out: *mut f32,
                                 n_out: usize, ggml_dtype: u32) -> c_int;
    pub fn gllmq_quantized_matmul_host(ctx: *mut gllmq_ctx, w: *const c_void, w_bytes: usize, x: *const f32,
                                       y: *mut f32, ggml_dtype: u32, m: usize, n: usize, k: usize) -> c_int;
}

/// Owner of one library context (one per device).  `Send + Sync` like the trait demands
/// (src/compat/mod.rs:77): every entry point takes the context's lock for the time it enqueues,
/// the device memory kernels use beyond inputs and outputs is kept per stream (calls on different
/// streams never share it, calls on one stream are ordered by the stream), the host-slice forms
/// synchronise before they return, and `gllmq_last_error` hands each thread its own copy.
pub struct HipQuant {
    ctx: *mut gllmq_ctx,
}
unsafe impl Send for HipQuant {}
unsafe impl Sync for HipQuant {}

/// `(group of layer i or None, number of groups)` of an open GGUF file: the layers grouped by
/// their per-layer quant-type signature as `MixedQuantPlan::group_of` holds them
/// (build_graph.inc.rs:388-470); `None` for the whole plan when every layer has the same signature.
///
/// # Safety
/// `g` must be a live handle from `gllmq_gguf_open`.
pub unsafe fn mixed_quant_group_of(g: *const c_void) -> Option<(Vec<Option<u32>>, usize)> {
    let layers = gllmq_gguf_layer_count(g);
    let mut group_of = vec![u32::MAX; layers];
    let groups = gllmq_gguf_mixed_quant_groups(g, group_of.as_mut_ptr(), layers);
    if groups == 0 {
        return None;
    }
    Some((group_of.into_iter().map(|v| if v == u32::MAX { None } else { Some(v) }).collect(), groups))
}

/// Mirrors gllm's `BackendError` variants used on this path
/// (src/engine/executor_types.rs:322-329).
#[derive(Debug, Clone)]
pub enum QuantError {
    Hip(String),
    Unimplemented(&'static str),
    Other(String),
}

impl HipQuant {
    pub fn new(device: i32) -> Result<Self, QuantError> {
        let mut ctx = std::ptr::null_mut();
        let rc = unsafe { gllmq_init(&mut ctx, device) };
        if rc != GLLMQ_OK {
            return Err(QuantError::Hip(format!("gllmq_init failed with status {rc}")));
        }
        Ok(Self { ctx })
    }

    fn check(&self, rc: c_int, what: &'static str) -> Result<(), QuantError> {
        if rc == GLLMQ_OK {
            return Ok(());
        }
        let msg = unsafe { CStr::from_ptr(gllmq_last_error(self.ctx)) }.to_string_lossy().into_owned();
        Err(match rc {
            GLLMQ_ERR_UNIMPLEMENTED => QuantError::Unimplemented(what),
            GLLMQ_ERR_HIP => QuantError::Hip(msg),
            _ => QuantError::Other(msg),
        })
    }

    /// `Backend::quantized_matmul` with host slices (the trait's signature); `ggml_dtype` is
    /// `quant_type_to_ggml_dtype(quant_type) as u32` (src/loader/adapter.rs:90-130).
    pub fn quantized_matmul(&self, weight_blocks: &[u8], input: &[f32], output: &mut [f32], ggml_dtype: u32,
                            m: usize, n: usize, k: usize) -> Result<(), QuantError> {
        if input.len() < m * k || output.len() < m * n {
            return Err(QuantError::Other("quantized_matmul: input/output shorter than m*k / m*n".into()));
        }
        let rc = unsafe {
            gllmq_quantized_matmul_host(self.ctx, weight_blocks.as_ptr().cast(), weight_blocks.len(), input.as_ptr(),
                                        output.as_mut_ptr(), ggml_dtype, m, n, k)
        };
        self.check(rc, "quantized_matmul")
    }

    /// `Backend::dequantize` with host slices.
    pub fn dequantize(&self, block_data: &[u8], output: &mut [f32], ggml_dtype: u32) -> Result<(), QuantError> {
        let rc = unsafe {
            gllmq_dequantize_host(self.ctx, block_data.as_ptr().cast(), block_data.len(), output.as_mut_ptr(),
                                  output.len(), ggml_dtype)
        };
        self.check(rc, "dequantize")
    }

    /// Device-resident form used by the executor: `w`, `x`, `y` are HIP device addresses of
    /// tensors the HIP backend already owns (src/compat/hip_backend.rs:141-156).
    ///
    /// # Safety
    /// The pointers must be valid device allocations of the stated sizes on this context's device.
    pub unsafe fn quantized_matmul_device(&self, w: *const c_void, w_bytes: usize, x: *const f32, y: *mut f32,
                                          ggml_dtype: u32, m: usize, n: usize, k: usize,
                                          stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_quantized_matmul(self.ctx, w, w_bytes, x, y, ggml_dtype, m, n, k, stream), "quantized_matmul")
    }

    /// `Op::QuantGather { quant_type, vocab_size, hidden_dim, scale }` over device tensors
    /// (src/arch/auto_graph_fragments/build_graph.inc.rs:203-211): `out[i] = scale * row ids[i]`.
    ///
    /// # Safety
    /// The pointers must be valid device allocations: `table` of `table_bytes`, `ids` of `count`
    /// u32, `out` of `count * hidden_dim` f32, on this context's device.
    pub unsafe fn quant_gather_device(&self, table: *const c_void, table_bytes: usize, ggml_dtype: u32,
                                      vocab_size: usize, hidden_dim: usize, ids: *const u32, count: usize,
                                      scale: Option<f32>, out: *mut f32, stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_quant_gather(self.ctx, table, table_bytes, ggml_dtype, vocab_size, hidden_dim, ids, count,
                                      scale.unwrap_or(1.0), out, stream), "quant_gather")
    }

    /// The dense feed-forward block of a layer over device tensors (gate_proj, up_proj, `Op::SwiGlu`,
    /// down_proj: src/arch/auto_graph_fragments/build_graph.inc.rs:1957-1995).
    ///
    /// # Safety
    /// All pointers must be valid device allocations of the stated sizes on this context's device.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn ffn_swiglu_device(&self, gate: *const c_void, up: *const c_void, gate_up_bytes_each: usize,
                                    dtype_gate_up: u32, down: *const c_void, down_bytes: usize, dtype_down: u32,
                                    x: *const f32, out: *mut f32, m: usize, hidden: usize, ffn: usize,
                                    stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_ffn_swiglu(self.ctx, gate, up, gate_up_bytes_each, dtype_gate_up, down, down_bytes, dtype_down,
                                    x, out, m, hidden, ffn, 0, stream), "ffn_swiglu")
    }

    /// `ExpertRouteTable::from_gate_logits` on the device (src/moe/routing.rs:100-160): gate logits
    /// `[tokens][experts]` in, the route table `gllmq_moe_matvec` takes out (`route_expert` and
    /// `route_weight` are `[tokens][top_k]`, `route_len` is `[tokens]`).
    ///
    /// # Safety
    /// All pointers are device pointers on this context's device with the sizes above.
    pub unsafe fn moe_route_device(&self, logits: *const f32, tokens: usize, experts: usize, top_k: usize,
                                   capacity_factor: f32, route_expert: *mut u32, route_weight: *mut f32,
                                   route_len: *mut u32, stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_moe_route(self.ctx, logits, tokens, experts, top_k, capacity_factor, route_expert, route_weight,
                                   route_len, std::ptr::null_mut(), std::ptr::null_mut(), std::ptr::null_mut(), stream),
                   "moe_route")
    }

    /// The routed experts' feed-forward blocks, summed per token with the router weights.  Gate, up
    /// and down are the expert tensors as the file stores them, `*_stride` the bytes from one
    /// expert's rows to the next.
    ///
    /// # Safety
    /// All pointers are device pointers on this context's device; the route table is the one
    /// `moe_route_device` writes.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn moe_matvec_device(&self, gate: *const c_void, gate_bytes: usize, gate_stride: usize,
                                    up: *const c_void, up_bytes: usize, up_stride: usize, dtype_gate_up: u32,
                                    down: *const c_void, down_bytes: usize, down_stride: usize, dtype_down: u32,
                                    x: *const f32, out: *mut f32, tokens: usize, hidden: usize, ffn: usize,
                                    experts: usize, top_k: usize, route_expert: *const u32, route_weight: *const f32,
                                    route_len: *const u32, relu_gate: bool, stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_moe_matvec(self.ctx, gate, gate_bytes, gate_stride, up, up_bytes, up_stride, dtype_gate_up,
                                    down, down_bytes, down_stride, dtype_down, x, out, tokens, hidden, ffn, experts,
                                    top_k, route_expert, route_weight, route_len, relu_gate as c_int, stream),
                   "moe_matvec")
    }

    /// `Op::Argmax` over device logits `[rows][ld]` (argmax_token, src/engine/executor_step.rs:48-55):
    /// `token[r]` is `u32::MAX` where the reference returns `None`.
    ///
    /// # Safety
    /// `logits` must hold `rows * ld` f32, `token` `rows` u32, `value` null or `rows` f32, on this device.
    pub unsafe fn argmax_device(&self, logits: *const f32, rows: usize, n: usize, ld: usize, token: *mut u32,
                                value: *mut f32, stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_argmax(self.ctx, logits, rows, n, ld, token, value, stream), "argmax")
    }

    /// `Backend<E>::quantized_matmul` for `E` = `half::f16` (`elem` 1) or `half::bf16` (`elem` 2) over
    /// device buffers of that element type (src/compat/mod.rs:376-378); 0 is f32.  Results are the
    /// f32 call's, rounded to the nearest element, ties to even (`E::from_f32`).
    ///
    /// # Safety
    /// `w` must hold `w_bytes` bytes, `x` `m * k` and `y` `m * n` elements of the type, on this device.
    pub unsafe fn quantized_matmul_elem_device(&self, w: *const c_void, w_bytes: usize, x: *const c_void, y: *mut c_void,
                                               ggml_dtype: u32, m: usize, n: usize, k: usize, elem: c_int,
                                               stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_quantized_matmul_elem(self.ctx, w, w_bytes, x, y, ggml_dtype, m, n, k, elem, stream),
                   "quantized_matmul")
    }

    /// `Op::QuantGather` into rows of element type `elem` (0 f32, 1 f16, 2 bf16): the f32 lookup's
    /// values rounded to the nearest element, ties to even.  `scale`: `None` for none.
    ///
    /// # Safety
    /// `table` must hold `table_bytes` bytes, `ids` `count` u32, `out` `count * hidden` elements of
    /// the type, all on this device.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn quant_gather_elem_device(&self, table: *const c_void, table_bytes: usize, ggml_dtype: u32,
                                           vocab_size: usize, hidden_dim: usize, ids: *const u32, count: usize,
                                           scale: Option<f32>, out: *mut c_void, elem: c_int,
                                           stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_quant_gather_elem(self.ctx, table, table_bytes, ggml_dtype, vocab_size, hidden_dim, ids, count,
                                           scale.unwrap_or(1.0), out, elem, stream), "quant_gather")
    }

    /// The dense feed-forward block over activations and outputs of element type `elem`; with
    /// `accumulate` it is added to `out` instead of replacing it (the `Op::Add` of a shared expert's
    /// block and of the residual, build_graph.inc.rs:2132-2170), one rounding to nearest even.
    ///
    /// # Safety
    /// As `ffn_swiglu_device`, with `x` and `out` holding `m * hidden` elements of the type.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn ffn_swiglu_elem_device(&self, gate: *const c_void, up: *const c_void, gate_up_bytes_each: usize,
                                         dtype_gate_up: u32, down: *const c_void, down_bytes: usize, dtype_down: u32,
                                         x: *const c_void, out: *mut c_void, m: usize, hidden: usize, ffn: usize,
                                         elem: c_int, accumulate: bool, relu_gate: bool,
                                         stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_ffn_swiglu_elem(self.ctx, gate, up, gate_up_bytes_each, dtype_gate_up, down, down_bytes,
                                         dtype_down, x, out, m, hidden, ffn, relu_gate as c_int, elem,
                                         if accumulate { GLLMQ_OUT_ACCUMULATE } else { 0 }, stream), "ffn_swiglu")
    }

    /// The routed experts' blocks over activations and outputs of element type `elem`, replacing
    /// `out` or added to it.
    ///
    /// # Safety
    /// As `moe_matvec_device`, with `x` and `out` holding `tokens * hidden` elements of the type.
    #[allow(clippy::too_many_arguments)]
    pub unsafe fn moe_matvec_elem_device(&self, gate: *const c_void, gate_bytes: usize, gate_stride: usize,
                                         up: *const c_void, up_bytes: usize, up_stride: usize, dtype_gate_up: u32,
                                         down: *const c_void, down_bytes: usize, down_stride: usize, dtype_down: u32,
                                         x: *const c_void, out: *mut c_void, tokens: usize, hidden: usize, ffn: usize,
                                         experts: usize, top_k: usize, route_expert: *const u32,
                                         route_weight: *const f32, route_len: *const u32, elem: c_int, accumulate: bool,
                                         relu_gate: bool, stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_moe_matvec_elem(self.ctx, gate, gate_bytes, gate_stride, up, up_bytes, up_stride, dtype_gate_up,
                                         down, down_bytes, down_stride, dtype_down, x, out, tokens, hidden, ffn, experts,
                                         top_k, route_expert, route_weight, route_len, relu_gate as c_int, elem,
                                         if accumulate { GLLMQ_OUT_ACCUMULATE } else { 0 }, stream), "moe_matvec")
    }

    /// Whether a chained launch since the last look ran out of its bounded wait (option
    /// "chain_dependent"); call after waiting for the stream.
    pub fn chain_status(&self) -> bool {
        unsafe { gllmq_chain_status(self.ctx) != 0 }
    }

    /// The lm_head matvec of one activation row and `Op::Argmax` behind it as one call.  `logits`
    /// may be null for Q6_K / Q8_0 matrices with `k <= 16384`: the logits then never reach memory.
    ///
    /// # Safety
    /// `w` must hold `w_bytes` bytes, `x` `k` f32, `logits` null or `n` f32, `token` one u32, `value`
    /// null or one f32, all on this device.
    pub unsafe fn lm_head_argmax_device(&self, w: *const c_void, w_bytes: usize, x: *const f32, ggml_dtype: u32, n: usize,
                                        k: usize, logits: *mut f32, token: *mut u32, value: *mut f32,
                                        stream: *mut c_void) -> Result<(), QuantError> {
        self.check(gllmq_lm_head_argmax(self.ctx, w, w_bytes, x, ggml_dtype, n, k, logits, token, value, stream),
                   "lm_head_argmax")
    }

    /// The same lookup with host slices (table uploaded, rows downloaded).
    pub fn quant_gather(&self, table: &[u8], ggml_dtype: u32, vocab_size: usize, hidden_dim: usize, ids: &[u32],
                        scale: Option<f32>, output: &mut [f32]) -> Result<(), QuantError> {
        if output.len() < ids.len() * hidden_dim {
            return Err(QuantError::Other("quant_gather: output shorter than ids.len() * hidden_dim".into()));
        }
        let rc = unsafe {
            gllmq_quant_gather_host(self.ctx, table.as_ptr().cast(), table.len(), ggml_dtype, vocab_size, hidden_dim,
                                    ids.as_ptr(), ids.len(), scale.unwrap_or(1.0), output.as_mut_ptr())
        };
        self.check(rc, "quant_gather")
    }
}

impl Drop for HipQuant {
    fn drop(&mut self) {
        unsafe { gllmq_destroy(self.ctx) }
    }
}
