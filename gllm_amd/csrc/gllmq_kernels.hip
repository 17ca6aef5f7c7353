// Single translation unit of every gfx950 kernel of the library.  It is compiled to a
// code object (hipcc --genco) that the host library embeds and loads with
// hipModuleLoadData; kernels are found by their extern "C" names.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_device.h"
#include "gq_params.h"

#include "dequant.hip.inc"
#include "gemv.hip.inc"
#include "gemv_i8.hip.inc"
#include "mm8.hip.inc"
#include "mm8_q6k.hip.inc"
#include "mm8_q8_0.hip.inc"
#include "mmf.hip.inc"
#include "mmf_q6k.hip.inc"
#include "mmf_q8_0.hip.inc"
#include "moe.hip.inc"
#include "argmax.hip.inc"
#include "ffn.hip.inc"
#include "route.hip.inc"
