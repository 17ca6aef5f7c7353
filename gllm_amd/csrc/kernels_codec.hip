// One of the translation units of the library's gfx950 kernels.  Each is compiled to a code
// object of its own (hipcc --genco), in parallel; the host library embeds them all and loads them
// with hipModuleLoadData; kernels are found by their extern "C" names.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "gq_device.h"
#include "gq_params.h"

#include "dequant.hip.inc"
#include "gemv.hip.inc"
#include "gemv_i8.hip.inc"
#include "argmax.hip.inc"
#include "ffn.hip.inc"
#include "route.hip.inc"
#include "convert.hip.inc"
#include "touch.hip.inc"
