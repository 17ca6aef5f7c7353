// One of the translation units of the library's gfx950 kernels.  Each is compiled to a code
// object of its own (hipcc --genco), in parallel; the host library embeds them all and loads them
// with hipModuleLoadData; kernels are found by their extern "C" names.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_device.h"
#include "gq_params.h"

// templates only: the kernels of these files are instantiated in another translation unit
#define GQ_TEMPLATES_ONLY
#include "gemv.hip.inc"
#include "gemv_i8.hip.inc"
#include "mm8.hip.inc"
#include "mm8_q6k.hip.inc"
#define GQ_Q6K_STEPWISE AREG // (115 -> 166 registers of 168, no scratch; the Q6_K down launch of 128 experts 93.1 -> 91.4 us)
#include "mm8s.hip.inc"
#undef GQ_TEMPLATES_ONLY

#include "moe.hip.inc"
