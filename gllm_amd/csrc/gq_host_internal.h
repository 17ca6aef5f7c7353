// Shared between the translation units of the host library; not part of the public ABI.
#ifndef GQ_HOST_INTERNAL_H
#define GQ_HOST_INTERNAL_H

#include "gllm_hip_quant.h"

// Records `message` as the context's last error and returns `status`.
extern "C" int gq_ctx_set_error(gllmq_ctx *ctx, int status, const char *message);

#endif
