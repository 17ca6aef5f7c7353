// Shared between the translation units of the host library; not part of the public ABI.
#ifndef GQ_HOST_INTERNAL_H
#define GQ_HOST_INTERNAL_H

#include "gllm_hip_quant.h"

#define GQ_INTERNAL __attribute__((visibility("hidden")))

// Records `message` as the context's last error and returns `status`.
extern "C" GQ_INTERNAL int gq_ctx_set_error(gllmq_ctx *ctx, int status, const char *message);

// Device of a context.
extern "C" GQ_INTERNAL int gq_ctx_device(const gllmq_ctx *ctx);

// gllmq_quantized_matmul with every byte of scratch taken from `block_dev` (`block_bytes` of
// device memory, 256-byte aligned, whose first GQ_BLOCK_ZEROED_BYTES are zero on the first call
// and are left zero by every call): nothing is allocated, and a shape that needs more scratch
// than the block holds fails with GLLMQ_ERR_BAD_SHAPE.
#define GQ_BLOCK_ZEROED_BYTES 4096
extern "C" GQ_INTERNAL int gq_quantized_matmul_on_block(gllmq_ctx *ctx, const void *w_dev, size_t w_bytes, const float *x_dev,
                                                        float *y_dev, uint32_t ggml_dtype, size_t m, size_t n, size_t k,
                                                        void *block_dev, size_t block_bytes, void *stream);

// Looks up, once per device, the address of the device array behind gllmq_quantized_matmul_noalloc
// (`device` must be current).  Called by gllmq_init, so that the entry point never has to.
extern "C" GQ_INTERNAL int gq_noalloc_init(gllmq_ctx *ctx, int device);

#endif
