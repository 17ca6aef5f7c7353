// One of the translation units of the library's gfx950 kernels: the streamed form of the int8
// matrix-core kernels (mm8s.hip.inc) for Q8_0, a code object of its own so that it builds beside
// the one of the K-quants.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_device.h"
#include "gq_params.h"

// templates only: the kernels of these files are instantiated in another translation unit
#define GQ_TEMPLATES_ONLY
#include "mm8.hip.inc"
#include "mm8_q6k.hip.inc"
#include "mm8_q8_0.hip.inc"
#undef GQ_TEMPLATES_ONLY

#define GQ_MM8S_Q8_0
#include "mm8s.hip.inc"
