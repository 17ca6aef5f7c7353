// One of the translation units of the library's gfx950 kernels.  Each is compiled to a code
// object of its own (hipcc --genco), in parallel; the host library embeds them all and loads them
// with hipModuleLoadData; kernels are found by their extern "C" names.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_device.h"
#include "gq_params.h"

// templates only: the kernels of this file are instantiated in another translation unit
#define GQ_TEMPLATES_ONLY
#include "mm8.hip.inc"
#include "mm8_q6k.hip.inc"
#include "mm8s.hip.inc"
#include "mmf.hip.inc"
#undef GQ_TEMPLATES_ONLY

#include "mmfs.hip.inc"
#include "mmfr.hip.inc"
