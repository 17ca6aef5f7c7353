// Host side of libgllm_hip_quant.so: the C ABI of include/gllm_hip_quant.h over the
// embedded gfx950 code objects.  Kernels are launched with hipModuleLaunchKernel on the
// caller's stream, the driver-style convention the reference's HIP backend uses
// (src/compat/hip_backend.rs:211-238), except that the module is loaded and every
// function resolved once per context instead of once per launch.
#include "gllm_hip_quant.h"
#include "gq_host_internal.h"
#include "gq_params.h"

#include <hip/hip_runtime_api.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <type_traits>
#include <unordered_map>
#include <unordered_set>
#include <vector>

// The code objects built from the kernels_*.hip translation units, placed in .rodata by the
// assembler (GLLMQ_HSACO_DIR is the build directory).
#define GLLMQ_EMBED(NAME)                                                              \
    __asm__(".section .rodata\n"                                                       \
            ".balign 4096\n"                                                           \
            ".global gllmq_co_" #NAME "\n"                                             \
            "gllmq_co_" #NAME ":\n"                                                    \
            ".incbin \"" GLLMQ_HSACO_DIR "/kernels_" #NAME ".hsaco\"\n"                 \
            ".byte 0\n"                                                                \
            ".previous\n");                                                            \
    extern "C" const unsigned char gllmq_co_##NAME[];
GLLMQ_EMBED(codec)
GLLMQ_EMBED(mm8)
GLLMQ_EMBED(mm8s)
GLLMQ_EMBED(mm8s_q8_0)
GLLMQ_EMBED(mm8c)
GLLMQ_EMBED(mm8_q6k_q8_0)
GLLMQ_EMBED(mmf)
GLLMQ_EMBED(mmfs)
GLLMQ_EMBED(moe)

namespace {

constexpr uint32_t T_Q8_0 = GLLMQ_TYPE_Q8_0, T_Q4_K = GLLMQ_TYPE_Q4_K, T_Q5_K = GLLMQ_TYPE_Q5_K,
                   T_Q6_K = GLLMQ_TYPE_Q6_K;

struct Format {
    uint32_t dtype;
    size_t block_size, block_bytes;
    size_t group_bytes; // bytes of 256 elements
    size_t w_align;
    const char *tag;
};

const Format kFormats[] = {
    { T_Q8_0, 32, 34, 272, 2, "q8_0" },
    { T_Q4_K, 256, 144, 144, 16, "q4k" },
    { T_Q5_K, 256, 176, 176, 16, "q5k" },
    { T_Q6_K, 256, 210, 210, 2, "q6k" },
};
constexpr int kNumFormats = 4;

const Format *find_format(uint32_t dtype)
{
    for (const Format &f : kFormats)
        if (f.dtype == dtype) return &f;
    return nullptr;
}

int format_index(uint32_t dtype)
{
    for (int i = 0; i < kNumFormats; ++i)
        if (kFormats[i].dtype == dtype) return i;
    return -1;
}

using gq::ArgmaxParams;
using gq::GatherParams;
using gq::GemvParams;
using gq::Mm8Params;
using gq::MmfParams;
using gq::MmfPrepParams;
using gq::MmfReduceParams;
using gq::Mm8ChainEntry;
using gq::Mm8ChainParams;
using gq::MoeActParams;
using gq::MoeCombineParams;
using gq::MoeGemvParams;
using gq::MoeJob;
using gq::MoeJob8;
using gq::MoeMm8Params;
using gq::MoePlanParams;

// Bytes of one block's activation image and of the GEMM's LDS, by 32-row activation tiles (1 or
// 2) and format (0 = Q4_K, 1 = Q5_K, 2 = Q6_K).
uint32_t mmf_image_bytes(uint32_t mt) { return mt == 1 ? gq::MmfLds<1>::image : gq::MmfLds<2>::image; }
uint32_t mmf_lds_bytes(uint32_t mt, int fmt)
{
    static const uint32_t kTotal[2][4] = {
        { gq::MmfLds<1, 0>::total, gq::MmfLds<1, 1>::total, gq::MmfLds<1, 2>::total, gq::MmfLds<1, 3>::total },
        { gq::MmfLds<2, 0>::total, gq::MmfLds<2, 1>::total, gq::MmfLds<2, 2>::total, gq::MmfLds<2, 3>::total },
    };
    return kTotal[mt - 1][fmt];
}

// Formats of the int8 matrix-core kernels, in the order of the kernel tables below.
// (the grouped MoE kernels exist for the first MM8_MOE_KINDS of them)
enum Mm8Kind { MM8_Q4K = 0, MM8_Q6K = 1, MM8_Q5K = 2, MM8_Q8_0 = 3, MM8_KINDS = 4, MM8_MOE_KINDS = 3 };
int mm8_kind(uint32_t dtype)
{
    return dtype == T_Q4_K ? MM8_Q4K : dtype == T_Q6_K ? MM8_Q6K : dtype == T_Q5_K ? MM8_Q5K : dtype == T_Q8_0 ? MM8_Q8_0 : -1;
}

// Bytes of LDS the int8 matrix-core kernels need: Q6_K keeps 16 sub-block sums per block
// instead of 8, Q8_0 none, and the weight stage of a wave differs by format.
uint32_t mm8_lds_bytes(uint32_t groups, uint32_t m, uint32_t pairs, int kind = MM8_Q4K)
{
    const uint32_t stage = kind == MM8_Q6K ? gq::MM8Q6_STAGE_BYTES : kind == MM8_Q8_0 ? gq::MM8Q8_STAGE_BYTES
                         : kind == MM8_Q5K ? gq::Mm8Format<1>::STAGE : gq::Mm8Format<0>::STAGE;
    return gq::mm8_lds_layout(groups, m, pairs, kind == MM8_Q6K ? 16u : kind == MM8_Q8_0 ? 0u : 8u, stage).total;
}

} // namespace

// Device memory beyond the inputs and outputs that the kernels of one call may use.  Every stream
// a context is used on gets its own set, so calls on different streams never share scratch and
// calls on one stream are ordered by the stream itself.
struct Scratch {
    hipStream_t stream = nullptr;
    uint64_t last_use = 0;
    bool fixed = false;          // carved from a block of fixed size: a call that needs more fails
    // K split of the int8 kernels: slice sums, and arrival counters that every launch leaves at 0
    float *mm8_part = nullptr;   // [MM8_SPLIT_PART_FLOATS]
    uint32_t *mm8_arrive = nullptr; // [MM8_SPLIT_MAX_LISTS]
    uint64_t *argmax_keys = nullptr; // [ARGMAX_MAX_ROWS][ARGMAX_MAX_PARTS]
    void *base = nullptr;        // the allocation that holds the three above
    void *mmf = nullptr;         // GEMM: activation images, then partial sums of K-split workgroups
    size_t mmf_bytes = 0;
    void *ffn = nullptr;         // gllmq_ffn_swiglu: gated activations, then gate/up results
    size_t ffn_bytes = 0;
    void *moe = nullptr;         // gllmq_moe_matvec: pair tables, jobs, intermediate activations
    size_t moe_bytes = 0;
    void *elem = nullptr;        // 16-bit activations and outputs as f32, for the kernels that do not convert themselves
    size_t elem_bytes = 0;
    void *box = nullptr;         // the chained launch's mailbox [kChainBoxPairs] of 64-bit words, zero when allocated
};

constexpr size_t kScratchArriveBytes = 4096; // MM8_SPLIT_MAX_LISTS words, padded; the chain kernel's counters behind them
constexpr size_t kLmHeadTicketAt = 600;      // the lm_head launch's count of finished workgroups
constexpr size_t kScratchKeysBytes = sizeof(uint64_t) * gq::ARGMAX_MAX_ROWS * gq::ARGMAX_MAX_PARTS;
constexpr size_t kScratchPartBytes = sizeof(float) * gq::MM8_SPLIT_PART_FLOATS;
constexpr size_t kScratchFixedBytes = kScratchArriveBytes + kScratchKeysBytes + kScratchPartBytes;
constexpr size_t kMaxScratchSlots = 16;

// Weights that a host-slice call uploaded, kept for the next call with the same slice
// (the reference keeps its uploaded weight blob the same way, src/compat/hip_backend.rs:141-156).
struct CachedWeights {
    const void *host = nullptr;
    size_t bytes = 0;
    void *dev = nullptr;
    uint64_t last_use = 0;
};

struct gllmq_ctx {
    int device = 0;
    hipModule_t modules[9] = {}; // one per embedded code object
    hipFunction_t dequant[kNumFormats][2] = {}; // [format][0 = scalar stores, 1 = float4 stores]
    hipFunction_t gather[kNumFormats][2] = {};  // quantized embedding lookup [format][0 = scalar stores, 1 = float4 stores]
    hipFunction_t gather_e16[kNumFormats][2] = {}; // the same into rows of a 16-bit element type [format][0 = scalar stores, 1 = 8-byte stores]
    hipFunction_t finish_elem = nullptr;        // f32 result in scratch -> output of any element type, plain or added to it
    // gated form of the int8 kernels (gate and up rows in one launch, act(gate) * up out):
    // [0 = Q4_K, 1 = Q5_K][pairs 1,2,4][early steps 1,2,4] and the register-operand variants
    hipFunction_t mm8_glu[2][3][3] = {};
    hipFunction_t mm8_gated_p4[MM8_KINDS] = {}; // five to eight rows of gated activations (a down projection's), by Mm8Kind
    hipFunction_t mm8_glu_areg[2][2][3][2] = {};
    hipFunction_t glu_act = nullptr;            // act(gate) * up as a kernel of its own
    hipFunction_t argmax_part = nullptr, argmax_final = nullptr;
    hipFunction_t dequant_wave = nullptr;       // Q4_K with 16-byte aligned blocks and outputs: one block per wave
    hipFunction_t dequant_wave_q5k = nullptr;   // the same for Q5_K
    hipFunction_t gemv[kNumFormats][2] = {};    // [format][m - 1], f32 multiply-add flavour
    hipFunction_t gemv_i8[kNumFormats][2] = {}; // [format][m - 1], integer-dot flavour (default)
    // call_mutex held: launches are only counted and the last kernel noted, nothing is enqueued
    // (gllmq_lm_head_argmax asks which kernel the one-row matmul of its shape would get)
    bool probe = false;
    uint32_t probe_launches = 0;
    hipFunction_t probe_fn = nullptr;
    hipFunction_t gemv_i8_argmax[kNumFormats] = {}; // one row, ending in the candidates of the greedy token choice
    // int8 matrix-core kernels [Mm8Kind][pairs 1,2,4][early steps 1,2,4], and the same with
    // register-resident activation operands [Mm8Kind][pairs 1,2][early][passes per tile - 1]
    hipFunction_t mm8[MM8_KINDS][3][3] = {};
    hipFunction_t mm8_areg[MM8_KINDS][2][3][2] = {};
    // streamed form (loader waves + arithmetic waves) [0 = Q4_K, 1 = Q5_K, 2 = Q6_K, 3 = Q8_0][variant]: register
    // operands p1_e1, p1_e2, p2_e4, then LDS operands p1_e2, p2_e4, p4_e4
    hipFunction_t mm8s[4][7] = {};
    bool use_mm8s = true;                       // "mm8s" = 0: the fetch-and-compute kernels throughout
    bool batch_overlap = true;                  // "batch_overlap" = 0: the kernels of a batch run strictly one after the other
    bool mm8s_all = false;                      // "mm8s_all" = 1: the streamed form wherever it fits, also where another was timed faster
    bool mm8_small_to_gemv = true;              // "mm8_small_to_gemv" = 0: one Q4_K row over few weight rows stays on the matrix-core kernels
    bool mm8s_areg = true;                      // "mm8s_areg" = 0: the streamed kernels never keep the digit planes in registers
    uint32_t mm8s_depth = 0;                    // "mm8s_depth": items a loader keeps unconfirmed, 0 = by item size
    uint32_t mm8s_min_rows = 8;                 // "mm8s_min_rows": fewest weight rows per CU that take the streamed form
    hipFunction_t moe_mm8_glu_fn[3][2] = {};    // gated gate/up kernels [Mm8Kind (Q4_K and Q5_K only)][passes per tile - 1]
    hipFunction_t mmf_q4k[4][2][2] = {};        // f16 matrix-core GEMM [0 = Q4_K, 1 = Q5_K, 2 = Q6_K, 3 = Q8_0][32-row activation tiles - 1][bf16 mode]
    hipFunction_t mmfs[2][2] = {};              // its streamed form [0 = Q4_K, 1 = Q5_K][bf16 mode]
    hipFunction_t mmfr[2] = {};                 // the streamed form whose waves prepare their own activations (f32, 9 to 16 rows) [0 = Q4_K, 1 = Q5_K]
    bool use_mmfr = true;                       // "mmfr" = 0: never
    uint32_t mmfr_min_rows = 8;                 // "mmfr_min_rows": fewest weight rows per CU that take it
    hipFunction_t mm8c[3][2][2] = {};           // chains of streamed matmuls in one launch [0 = Q4_K, 1 = Q5_K, 2 = Q8_0][some entry in pairs of blocks][some entry waits for the one before it]
    bool chain_dependent = false;               // "chain_dependent" = 1: an entry that reads the output of the one before it stays in the chained launch (measured slower than a launch of its own)
    uint32_t chain_epoch = 1;                   // epochs handed to chained entries so far (see Mm8ChainParams::box)
    bool use_chain = true;                      // "chain" = 0: every entry of a batch is a launch of its own
    uint32_t chain_min_rows = 1;                // "chain_min_rows": fewest weight rows in a CU's share of an entry that joins a chain
    uint32_t chain_spin_limit = 1u << 20;       // "chain_spin_limit": polls of a dependency counter before a workgroup gives up
    uint32_t *chain_error = nullptr;            // host memory the device can write: set when such a wait ran out
    bool mmfs_all = false;                      // "mmfs_all" = 1: the streamed GEMM wherever it fits, also where the other form was timed faster
    bool use_mmfs = true;                       // "mmfs" = 0: the three-launch GEMM throughout
    uint32_t mmfs_min_rows = 8;                 // "mmfs_min_rows": fewest weight rows per CU that take the streamed GEMM
    hipFunction_t mmf_prep_lanes = nullptr;     // the images of the streamed form
    hipFunction_t mmf_prep[2] = {};             // its activation preparation [32-row activation tiles - 1]
    hipFunction_t mmf_reduce = nullptr;         // and the in-order sum of its K-split partial results
    hipFunction_t moe_plan = nullptr, moe_act = nullptr, moe_combine = nullptr, moe_route = nullptr;
    hipFunction_t moe_gemv[kNumFormats] = {};
    hipFunction_t moe_mm8_fn[MM8_KINDS][2] = {}; // grouped int8 matrix-core kernels [Mm8Kind][passes per tile - 1]
    hipFunction_t moe_mm8_q6k_rows = nullptr;   // Q6_K rows of at most 8 blocks: a wave per 32-row tile
    hipFunction_t moe_mm8s_fn[MM8_MOE_KINDS][2] = {}; // the grouped kernels in the streamed form [Mm8Kind][plain, gated]
    uint32_t *identity_rows = nullptr;          // device: 0..7, the activation rows of an ungathered matmul

    // Kernel-family choices (gllmq_set_option).  The defaults are the measured best; the tests
    // switch them to reach every kernel family through the public entry points.
    bool gemv_f32 = false;                      // "gemv_f32": the f32 multiply-add GEMV instead of the integer-dot one
    bool use_mm8 = true;                        // "mm8" = 0: no int8 matrix-core kernels
    bool use_mmf = true;                        // "mmf" = 0: more than 8 rows run 8-row passes
    bool ffn_fused = true;                      // "ffn_fused" = 0: gllmq_ffn_swiglu never uses the gated kernels
    // Fewest activation rows that send a format to the int8 matrix-core kernel (below, the GEMV
    // kernels are as fast or faster); 1 = always, 0 = never.
    uint32_t mm8_q6k_min_m = 3, mm8_q5k_min_m = 2, mm8_q8_0_min_m = 3;
    // Fewest rows the GEMM takes when the 8-row kernel would need more than one pass over the
    // weights (long rows: the prepared activations of all rows do not fit the LDS of a CU); 0 = never.
    uint32_t mmf_small_min_m = 3;
    uint32_t mm8_ksplit_max = 8;                // "mm8_ksplit": most slices of the K split (0 or 1 = never split)
    bool moe_mm8 = true;                        // "moe_mm8" = 0: expert rows stay on the GEMV kernels
    bool moe_mm8_q6k = true;                    // "moe_mm8_q6k" = 0: Q6_K expert rows stay there
    bool moe_glu = true;                        // "moe_glu" = 0: gate/up results to memory, activation as a kernel of its own
    uint32_t moe_slices = 0;                    // "moe_slices": workgroups that share a job's row tiles (0 = by the number of pairs and experts)
    bool moe_mm8_rows = true;                   // "moe_mm8_rows" = 0: no wave-per-tile kernel for short Q6_K rows
    uint32_t moe_streamed = 1;                  // "moe_streamed": the grouped kernels in the streamed form: 0 never, 1 while experts see few tokens each, 2 always
    uint32_t moe_depth = 0;                     // "moe_depth": items a loader of the streamed grouped kernels keeps unconfirmed (0 = as the dense launches)

    // One lock over every enqueue on this context: calls from several threads take turns on the
    // host (the kernels they enqueue overlap as their streams allow).
    // State of gllmq_quantized_matmul_batch while it enqueues (see launch2d).
    struct Overlap {
        bool on = false;                 // inside a batch
        bool entry_first = false;        // the next launch is the first of its entry
        bool group_open = false;         // a launch of this batch has been enqueued
        bool group_uses_scratch = false; // a kernel that may still be running uses the scratch
    } overlap;
    std::recursive_mutex call_mutex;
    std::vector<Scratch> scratch;               // one set per stream the context has been used on
    uint64_t use_counter = 0;
    std::vector<CachedWeights> weights;         // host-slice calls: uploaded weights by (pointer, length)
    size_t weights_cache_limit = size_t(64) << 30; // bytes kept before the least recently used goes
    uint64_t weight_uploads = 0;                // how many host-to-device weight copies the cache has done
    std::unordered_map<hipFunction_t, std::string> kernel_names;
    hipFunction_t last_kernel = nullptr;
    int num_cus = 256;
    uint32_t gemv_waves = 2048; // waves a GEMV launch aims to put on the device
    bool lm_head_fused = true;  // lm_head_argmax: candidates from the GEMV's own workgroups
    uint32_t call_elem = 0;     // element type of x and y of the matmul being enqueued (call_mutex held); 0 = f32
    // activations of the matmul being enqueued that are a gated product: x[r][i] = act(x[r][i]) * x[r][i + call_glu_off],
    // rows call_ldx elements apart (the input of a feed-forward block's down projection); 0 = plain
    uint32_t call_glu = 0, call_glu_off = 0, call_ldx = 0;
    bool ffn_glu_load = true;   // "ffn_glu_load" = 0: the gate activation always runs as a kernel of its own
    hipFunction_t mm8s_gated[2][6] = {};        // streamed gate/up kernels with act(g) * u at the end of a tile pair [Q4_K, Q5_K][p1_e1_a, p1_e2_a, p2_e4_a, p1_e2, p2_e4, p1_e4]
    bool ffn_streamed = true;                   // "ffn_streamed" = 0: gllmq_ffn_swiglu never uses them
    hipFunction_t mm8s_e16[4][6] = {};          // streamed kernels over 16-bit activations and outputs [format][p1_e1_a, p1_e2_a, p2_e4_a, p1_e2, p2_e4, p1_e4]
    hipFunction_t mm8s_glu[4][4] = {};          // streamed kernels that take gated activations [format][p1_e2, p2_e4, p1_e4, p4_e4]
    // streamed kernels whose items are pairs of blocks of a tile of at most 16 weight rows (one
    // activation row) [format][p1_e1_a, p1_e2_a, p1_e2, p1_e4, p1_e2 and p1_e4 over gated activations,
    // the first four over a 16-bit element type]
    hipFunction_t mm8s_fold[4][10] = {};
    // streamed kernels whose workgroups share a row range and take a slice of K each (two to four
    // activation rows over few weight rows) [format][p1_e4, p2_e4][plain, gated activations]
    hipFunction_t mm8s_split[4][2][2] = {};
    bool mm8s_q8_0 = true;                      // "mm8s_q8_0" = 0: Q8_0 never takes the streamed form
    bool mm8s_split_on = true;                  // "mm8s_split" = 0: such shapes stay on the fetch-and-compute form
    bool mm8s_fold_on = true;                   // "mm8s_fold" = 0: such tiles go block by block, half of the matrix-core columns idle
    hipFunction_t gemv_i8_glu[kNumFormats][2] = {};
    hipFunction_t gemv_i8_e16[kNumFormats][2] = {}; // the integer-dot GEMV over 16-bit activations and outputs
    bool elem_fused = true;     // "elem_fused" = 0: 16-bit elements always through conversion launches
    hipFunction_t convert_elem = nullptr;
    // Weight prefetch beside the dependent launches of a batch (touch.hip.inc).  Launches that
    // take part are numbered per context; a kernel of `announces` raises *progress to its number
    // when it starts, and the prefetch launch, on a stream of the context's own, reads the weights
    // of launch s while launch s - 1 runs.
    bool prefetch = false;                      // "prefetch" = 1: on (measured slower: the prefetch shares every CU's memory pipeline with the launch it runs beside)
    uint32_t prefetch_wgs = 0;                  // "prefetch_wgs": workgroups of the prefetch launch (0 = one per CU)
    uint32_t prefetch_threads = 64;             // "prefetch_threads": threads of each (64 .. 256)
    uint32_t prefetch_timeout_us = 200;         // "prefetch_timeout_us": longest wait for the launch before an entry's
    uint32_t prefetch_flags = 0;                // "prefetch_flags": TouchParams::flags
    bool prefetch_announce = true;              // "prefetch_announce" = 0: the launches stay silent (for measurements)
    uint32_t prefetch_min_kib = 4096;           // "prefetch_min_kib": smallest weight matrix worth a prefetch
    hipFunction_t touch = nullptr;
    hipStream_t side_stream = nullptr;
    hipEvent_t side_event = nullptr;
    unsigned long long *progress = nullptr;     // device
    unsigned long long launch_seq = 0;          // number of the last launch that was given one
    unsigned long long call_seq = 0;            // number the launch being enqueued announces itself under (0: none)
    std::unordered_set<hipFunction_t> announces;
    std::mutex err_mutex;
    std::string err;
};

namespace {

int fail(gllmq_ctx *ctx, int code, const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    if (ctx) {
        std::lock_guard<std::mutex> g(ctx->err_mutex);
        ctx->err = buf;
    }
    return code;
}

} // namespace

extern "C" int gq_ctx_set_error(gllmq_ctx *ctx, int status, const char *message)
{
    return fail(ctx, status, "%s", message ? message : "");
}

extern "C" int gq_ctx_device(const gllmq_ctx *ctx) { return ctx ? ctx->device : -1; }

namespace {

#define GLLMQ_HIP(ctx, call)                                                                  \
    do {                                                                                      \
        hipError_t e_ = (call);                                                               \
        if (e_ != hipSuccess)                                                                 \
            return fail(ctx, GLLMQ_ERR_HIP, "%s failed: %s", #call, hipGetErrorString(e_));   \
    } while (0)

int get_function(gllmq_ctx *ctx, hipFunction_t *f, const char *name)
{
    hipError_t e = hipErrorNotFound;
    for (hipModule_t mod : ctx->modules) {
        if (!mod) continue;
        e = hipModuleGetFunction(f, mod, name);
        if (e == hipSuccess) break;
        (void)hipGetLastError();
    }
    if (e != hipSuccess)
        return fail(ctx, GLLMQ_ERR_HIP, "kernel %s missing from the code objects: %s", name,
                    hipGetErrorString(e));
    ctx->kernel_names[*f] = name;
    return GLLMQ_OK;
}

bool stream_is_capturing(void *stream)
{
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

void carve_fixed(Scratch &S, void *base)
{
    uint8_t *b = static_cast<uint8_t *>(base);
    S.mm8_arrive = reinterpret_cast<uint32_t *>(b);
    S.argmax_keys = reinterpret_cast<uint64_t *>(b + kScratchArriveBytes);
    S.mm8_part = reinterpret_cast<float *>(b + kScratchArriveBytes + kScratchKeysBytes);
}

void free_scratch(Scratch &S)
{
    if (S.fixed) return;
    if (S.base) (void)hipFree(S.base);
    if (S.mmf) (void)hipFree(S.mmf);
    if (S.ffn) (void)hipFree(S.ffn);
    if (S.moe) (void)hipFree(S.moe);
    if (S.elem) (void)hipFree(S.elem);
    if (S.box) (void)hipFree(S.box);
    S = Scratch{};
}

// The scratch set of `stream` on this context (call_mutex held).  A stream the context has not
// seen gets a new set; beyond kMaxScratchSlots streams the least recently used set is given up
// after the device has drained.  Allocating is not possible while `stream` is being captured.
int acquire_scratch(gllmq_ctx *ctx, void *stream, Scratch **out)
{
    ++ctx->use_counter;
    for (Scratch &S : ctx->scratch)
        if (S.stream == static_cast<hipStream_t>(stream)) {
            S.last_use = ctx->use_counter;
            *out = &S;
            return GLLMQ_OK;
        }
    if (stream_is_capturing(stream))
        return fail(ctx, GLLMQ_ERR_INVALID,
                    "the context has no scratch for this stream yet and cannot allocate it during stream capture: "
                    "call gllmq_reserve (or run the call once) on this stream before capturing");
    GLLMQ_HIP(ctx, hipSetDevice(ctx->device));
    if (ctx->scratch.size() >= kMaxScratchSlots) {
        size_t lru = 0;
        for (size_t i = 1; i < ctx->scratch.size(); ++i)
            if (ctx->scratch[i].last_use < ctx->scratch[lru].last_use) lru = i;
        GLLMQ_HIP(ctx, hipDeviceSynchronize()); // its stream may be gone: wait for everything
        free_scratch(ctx->scratch[lru]);
        ctx->scratch.erase(ctx->scratch.begin() + static_cast<long>(lru));
    }
    Scratch S;
    S.stream = static_cast<hipStream_t>(stream);
    S.last_use = ctx->use_counter;
    GLLMQ_HIP(ctx, hipMalloc(&S.base, kScratchFixedBytes));
    hipError_t e = hipMemset(S.base, 0, kScratchArriveBytes);
    if (e != hipSuccess) {
        (void)hipFree(S.base);
        return fail(ctx, GLLMQ_ERR_HIP, "scratch: %s", hipGetErrorString(e));
    }
    carve_fixed(S, S.base);
    ctx->scratch.push_back(S);
    *out = &ctx->scratch.back();
    return GLLMQ_OK;
}

// Makes *buf hold at least `need` bytes.  Growing waits for the stream's earlier work (which may
// still use the old buffer; other streams have their own scratch), so it cannot happen while the
// stream is being captured, and never happens for a set of fixed size.
int grow_scratch(gllmq_ctx *ctx, const Scratch &S, void **buf, size_t *have, size_t need, void *stream, const char *what)
{
    if (*have >= need || ctx->probe) return GLLMQ_OK; // (a dry run of the dispatch allocates nothing)
    if (S.fixed)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "%s needs %zu bytes of scratch, the fixed scratch of this entry point has %zu",
                    what, need, *have);
    if (stream_is_capturing(stream))
        return fail(ctx, GLLMQ_ERR_INVALID,
                    "%s needs %zu bytes of scratch (the stream has %zu) and cannot allocate during stream capture: "
                    "call gllmq_reserve (or run the shape once) on this stream before capturing", what, need, *have);
    GLLMQ_HIP(ctx, hipSetDevice(ctx->device));
    if (*buf) {
        GLLMQ_HIP(ctx, hipStreamSynchronize(static_cast<hipStream_t>(stream)));
        GLLMQ_HIP(ctx, hipFree(*buf));
        *buf = nullptr;
        *have = 0;
    }
    GLLMQ_HIP(ctx, hipMalloc(buf, need));
    *have = need;
    return GLLMQ_OK;
}

// `uses_scratch`: the kernel reads or writes the stream's scratch.
// Inside a batch of independent matmuls (ctx->overlap.on) the first launch of an entry is enqueued
// without the order that a stream otherwise imposes on its kernels, so that it may start while
// the kernels of earlier entries are still running (the gap between two kernels and the first and
// last microsecond of each, when few CUs stream, are what a decode layer's matmuls lose most to).
// Everything else is an ordinary launch, which starts after all earlier work of the stream has
// finished, unordered launches included.  Two kernels that use the scratch never overlap.
int launch2d(gllmq_ctx *ctx, hipFunction_t f, uint32_t grid_x, uint32_t grid_y, uint32_t block, uint32_t lds,
             void *stream, void *params, size_t params_size, bool uses_scratch = false)
{
    if (ctx->probe) {
        ++ctx->probe_launches;
        ctx->probe_fn = f;
        return GLLMQ_OK;
    }
    void *config[] = { HIP_LAUNCH_PARAM_BUFFER_POINTER, params, HIP_LAUNCH_PARAM_BUFFER_SIZE,
                       &params_size, HIP_LAUNCH_PARAM_END };
    gllmq_ctx::Overlap &ov = ctx->overlap;
    // (the launch without order takes the launch's size in threads as 32-bit numbers)
    const bool unordered = ov.on && ov.entry_first && ov.group_open && !(uses_scratch && ov.group_uses_scratch) &&
                           static_cast<uint64_t>(grid_x) * block <= 0xFFFFFFFFull;
    if (unordered) {
        GLLMQ_HIP(ctx, hipExtModuleLaunchKernel(f, grid_x * block, grid_y, 1, block, 1, 1, lds, static_cast<hipStream_t>(stream),
                                                nullptr, config, nullptr, nullptr, hipExtAnyOrderLaunch));
    } else {
        GLLMQ_HIP(ctx, hipModuleLaunchKernel(f, grid_x, grid_y, 1, block, 1, 1, lds, static_cast<hipStream_t>(stream),
                                             nullptr, config));
        ov.group_uses_scratch = false; // it waits for everything before it
    }
    ov.group_open = true;
    ov.entry_first = false;
    ov.group_uses_scratch = ov.group_uses_scratch || uses_scratch;
    ctx->last_kernel = f;
    return GLLMQ_OK;
}

int launch(gllmq_ctx *ctx, hipFunction_t f, uint32_t grid, uint32_t block, uint32_t lds, void *stream,
           void *params, size_t params_size, bool uses_scratch = false)
{
    return launch2d(ctx, f, grid, 1, block, lds, stream, params, params_size, uses_scratch);
}

bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// Element `index` of activations or outputs whose element type is that of the call being enqueued
// (pointers are typed for the f32 case).
template <class T>
T *elem_at(const gllmq_ctx *ctx, T *base, size_t index)
{
    typedef typename std::conditional<std::is_const<T>::value, const uint8_t, uint8_t>::type Byte;
    return reinterpret_cast<T *>(reinterpret_cast<Byte *>(base) + index * (ctx->call_elem ? 2u : 4u));
}

// Elements between activation rows of the matmul being enqueued: k unless the caller says otherwise.
uint32_t row_stride_x(const gllmq_ctx *ctx, size_t k) { return ctx->call_ldx ? ctx->call_ldx : static_cast<uint32_t>(k); }

// What a kernel family answers when it would take the shape but cannot read gated activations:
// the caller then applies the gate in a launch of its own.
constexpr int kNeedPlainActivations = -2;

// Gated activations are read as aligned float4 from both factors.
bool glu_vector_ok(const gllmq_ctx *ctx) { return ctx->call_glu_off % 4u == 0u && ctx->call_ldx % 4u == 0u; }

// Shape-dependent fields of a GEMV launch over at most 64 groups (16384 elements) of K and
// m <= 2: how a row is split over lanes and waves, rows per workgroup, LDS.  `target_waves`
// is the number of waves the launch aims to put on the device.
struct GemvPlan {
    GemvParams P;
    uint32_t grid, threads, lds;
};

GemvPlan plan_gemv(const gllmq_ctx *ctx, uint32_t m, uint32_t n, uint32_t k, size_t row_bytes, uint32_t target_waves)
{
    GemvPlan L{};
    GemvParams &P = L.P;
    P.n = n;
    P.k = k;
    P.groups = (k + 255u) / 256u;
    P.row_bytes = static_cast<uint32_t>(row_bytes);
    const uint32_t parts = 4 * P.groups;
    if (parts >= 64) {
        P.ks = (parts + 63) / 64;
        P.rps = 1;
    } else {
        P.ks = 1;
        P.rps = 64 / parts;
    }
    const uint32_t rgs = std::max(1u, 4u / P.ks);
    const uint32_t nwaves = P.ks * rgs;
    const uint32_t row_steps = (n + P.rps - 1) / P.rps;
    uint32_t wgs = std::max(1u, target_waves / nwaves);
    wgs = std::min(wgs, (row_steps + rgs - 1) / rgs);
    uint32_t steps_per_wg = (row_steps + wgs * rgs - 1) / (wgs * rgs);
    P.rows_per_wg = steps_per_wg * rgs * P.rps;
    // partial sums of a K-split row meet in LDS: keep them within 8 KiB
    const uint32_t max_rows = 8192u / (4u * P.ks * m);
    if (P.ks > 1 && P.rows_per_wg > max_rows) P.rows_per_wg = std::max(rgs, max_rows / rgs * rgs);
    L.grid = (n + P.rows_per_wg - 1) / P.rows_per_wg;
    L.threads = 64 * nwaves;
    // integer-dot flavour: per part and activation row 48 plane words + 1 scale + 4 sums
    P.prep_words = ctx->gemv_f32 ? 0u : 53u * m * parts;
    L.lds = P.prep_words * 4u + (P.ks > 1 ? P.rows_per_wg * P.ks * m * 4u : 0u);
    return L;
}

int launch_gemv(gllmq_ctx *ctx, const Format &f, const uint8_t *w, size_t row_bytes, const float *x,
                float *y, uint32_t m, uint32_t n, uint32_t k, uint32_t ldx, uint32_t ldy, bool accumulate,
                bool act_bf16, void *stream)
{
    GemvPlan L = plan_gemv(ctx, m, n, k, row_bytes, ctx->gemv_waves);
    GemvParams &P = L.P;
    P.w = w;
    P.x = x;
    P.y = y;
    P.ldx = ldx;
    P.ldy = ldy;
    P.x_vec = aligned(x, 16) && (m == 1 || ldx % (ctx->call_elem ? 8 : 4) == 0);
    P.accumulate = accumulate ? 1u : 0u;
    P.act_bf16 = act_bf16 ? 1u : 0u;
    P.elem = ctx->call_elem;
    P.glu = ctx->call_glu;
    P.glu_off = ctx->call_glu_off;
    const int fi = format_index(f.dtype);
    hipFunction_t fn = ctx->gemv_f32 ? ctx->gemv[fi][m - 1]
                     : ctx->call_glu ? ctx->gemv_i8_glu[fi][m - 1]
                     : ctx->call_elem ? ctx->gemv_i8_e16[fi][m - 1]
                                      : ctx->gemv_i8[fi][m - 1];
    return launch(ctx, fn, L.grid, L.threads, L.lds, stream, &P, sizeof P);
}

int check_matmul_args(gllmq_ctx *ctx, const Format *f, const void *w, size_t w_bytes, const float *x,
                      float *y, uint32_t dtype, size_t m, size_t n, size_t k)
{
    if (!f)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "quantized_matmul: ggml dtype %u is not covered (supported: Q8_0=8, Q4_K=12, Q5_K=13, Q6_K=14)",
                    dtype);
    if (m == 0 || n == 0) return GLLMQ_OK;
    if (!w || !x || !y) return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul: NULL device pointer");
    if (k == 0) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quantized_matmul: k = 0");
    if (n > 0x7FFFFFFFu || k > 0x7FFFFFFFu || m > 0x7FFFFFFFu)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quantized_matmul: dimension exceeds 2^31-1");
    const size_t rb = gllmq_row_bytes(dtype, k);
    // the kernels address a workgroup's rows with 32-bit byte offsets from the first of them
    if (rb > (size_t(1) << 26))
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quantized_matmul: rows of %zu bytes (k=%zu) exceed the supported 64 MiB", rb, k);
    if (w_bytes < n * rb)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE,
                    "quantized_matmul: weight buffer has %zu bytes, n=%zu rows of k=%zu need %zu", w_bytes, n, k,
                    n * rb);
    if (!aligned(w, f->w_align) || (rb % f->w_align) != 0)
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "quantized_matmul: weights of %s must be %zu-byte aligned",
                    f->tag, f->w_align);
    if (!aligned(x, 4) || !aligned(y, 4))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "quantized_matmul: activations and outputs must be 4-byte aligned");
    return -1; // go on
}

// Q4_K and Q5_K with up to 8 rows in the streamed form (mm8s.hip.inc): taken when the weight rows
// give every CU at least one 32-row tile, one pass over the weights serves all activation rows and
// the LDS ring holds enough items.  Returns -1 when the shape is not for it.
// `w2` != null selects the gated form: `w` holds the n gate rows, `w2` the n up rows, and
// y = act(gate . x) * (up . x) (Q4_K and Q5_K, up to four activation rows).
// `S` != null lets few weight rows under two to four rows of long activations share a row range
// among workgroups, a slice of K each (the sums meet in S->mm8_part).
int run_mm8s(gllmq_ctx *ctx, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n, size_t k,
             bool act_bf16, void *stream, const uint8_t *w2 = nullptr, bool glu_relu = false, Scratch *S = nullptr)
{
    const int kind = mm8_kind(f.dtype);
    const bool glu = w2 != nullptr;
    if (glu && ((kind != MM8_Q4K && kind != MM8_Q5K) || m > 4 || ctx->call_glu || ctx->call_elem)) return -1;
    if (!ctx->use_mm8 || !ctx->use_mm8s || (kind != MM8_Q4K && kind != MM8_Q5K && kind != MM8_Q6K && kind != MM8_Q8_0) || m == 0 || m > 8) return -1;
    if (kind == MM8_Q5K && ctx->mm8_q5k_min_m == 0) return -1;
    if (kind == MM8_Q6K && ctx->mm8_q6k_min_m == 0) return -1;
    // Q8_0: an item is a group of 8 blocks, so rows of whole groups only
    if (kind == MM8_Q8_0 && (ctx->mm8_q8_0_min_m == 0 || !ctx->mm8s_q8_0 || k % 256 != 0)) return -1;
    const int sfmt = kind == MM8_Q8_0 ? 3 : kind == MM8_Q6K ? 2 : kind == MM8_Q5K ? 1 : 0;
    const uint32_t pieces = sfmt == 3 ? gq::Mm8sFormat<3>::PIECES : sfmt == 2 ? gq::Mm8sFormat<2>::PIECES : sfmt == 1 ? gq::Mm8sFormat<1>::PIECES : gq::Mm8sFormat<0>::PIECES;
    const uint32_t subs = sfmt == 3 ? 0u : sfmt == 2 ? 16u : 8u;
    if (!aligned(x, 16) || k % 8 != 0) return -1;
    const uint32_t cus = static_cast<uint32_t>(ctx->num_cus);
    const uint32_t groups = static_cast<uint32_t>((k + 255) / 256), tiles = static_cast<uint32_t>((n + 31) / 32);
    // Every CU gets its share of the rows, as tiles of equal height; with fewer than 32 rows per CU
    // the tiles are lower than the 32 rows the matrix cores multiply, which costs nothing here (the
    // stream bounds the kernel).  Below `mm8s_min_rows` rows per CU the K split of the other form,
    // which keeps whole tiles and shares their blocks between CUs, is left to do it.
    // (two rows and more: from 4 rows per CU, where the K split of the other form and the GEMV are
    // behind: 2 x 4096 -> 1024 Q4_K 5.1-5.4 against 5.9-6.1 and 5.5-5.7 us)
    // (one row, in pairs of blocks: likewise from 4 rows per CU, 8192 -> 1536 Q4_K 5.8 against 7.3 us,
    // 14336 -> 1024 6.8 against 9.1, Q6_K 8.7 against 11.8)
    const bool may_fold = ctx->mm8s_fold_on && m == 1 && !glu;
    const uint32_t min_rows = (m >= 2 || may_fold) ? std::min(ctx->mm8s_min_rows, 4u) : ctx->mm8s_min_rows;
    if (n < static_cast<size_t>(min_rows) * cus) return -1;
    const uint32_t mm = static_cast<uint32_t>(m), pi = mm <= 2 ? 0u : (mm <= 4 ? 1u : 2u), pairs = 1u << pi;
    // K split: two to four activation rows of at least 32 blocks over 32-row tiles for at most half
    // of the CUs.  Every workgroup prepares the activations it multiplies, so whole rows of K per
    // workgroup cost rows x K of preparation in each (and four rows of 14336 do not fit the LDS);
    // `ksplit` workgroups share a tile and take a slice of at least 16 blocks each.
    uint32_t ksplit = 1;
    // (Q6_K: two rows; with three and four the fetch-and-compute form stays ahead, 14336 -> 4096 at
    // three rows 19.8 against 22.5 us)
    if (S && ctx->mm8s_split_on && !glu && !ctx->call_elem && mm >= 2 && mm <= (kind == MM8_Q6K && !ctx->mm8s_all ? 2u : 4u) &&
        groups >= 32 && tiles * 2u <= cus && tiles <= gq::MM8_SPLIT_MAX_LISTS)
        ksplit = std::min(cus / tiles, groups / 16u);
    while (ksplit > 1 && static_cast<size_t>(ksplit) * mm * n > gq::MM8_SPLIT_PART_FLOATS) --ksplit;
    // (slices for fewer than three quarters of the CUs leave too many of them idle: Q8_0 8192 -> 1024
    // at two rows 10.9 against 9.6 us for the GEMV)
    if (ksplit > 1 && !ctx->mm8s_all && ksplit * tiles * 4u < cus * 3u) ksplit = 1;
    const bool split = ksplit > 1;
    const uint32_t kslice = (groups + ksplit - 1u) / ksplit, lds_groups = split ? kslice : groups; // blocks a workgroup prepares
    const uint32_t rows_per_wg = split ? 32u : static_cast<uint32_t>((n + cus - 1) / cus);
    const uint32_t grid = static_cast<uint32_t>((n + rows_per_wg - 1) / rows_per_wg);
    const uint32_t wg_tiles = (rows_per_wg + 31u) / 32u, tile_rows = (rows_per_wg + wg_tiles - 1u) / wg_tiles;
    // One activation row over tiles of at most 16 weight rows: an item is a pair of blocks of the
    // tile, so that all 32 columns of the matrix cores carry weights (14336 -> 4096 is bound by the
    // arithmetic, not by the stream, when half of them idle).
    const bool fold = may_fold && tile_rows <= 16 && groups > 8; // (up to 8 blocks there is nothing to pair: a block per wave)
    if (may_fold && !fold && n < static_cast<size_t>(ctx->mm8s_min_rows) * cus) return -1;
    const uint32_t ipt = fold ? gq::mm8s_fold_pairs(groups) : lds_groups; // items per tile
    const uint32_t item_bytes = (fold ? 2u : 1u) * tile_rows * pieces * 16u; // a row of an item in LDS: its 16-byte pieces side by side
    const uint32_t fixed = gq::mm8s_lds_layout(lds_groups, mm, pairs, item_bytes, 0, subs, glu).total;
    const uint32_t items = (glu ? 2u : 1u) * wg_tiles * ipt; // (gated: a gate tile and an up tile per tile of rows)
    uint32_t slots = std::min(items, (160u * 1024u - std::min(fixed, 160u * 1024u)) / item_bytes);
    if (slots < items) slots -= slots % gq::MM8S_LOADERS; // a reused ring is a whole number of rounds of the loaders
    // Items a loader keeps unconfirmed.  One or two activation rows: one item (the wave requests an
    // item, waits for the one before it and confirms that: an arithmetic wave sees an item as soon
    // as it is there; with more outstanding the stream got no faster and the items later: one row
    // 4096 -> 4096 5.30 against 5.95 us, 4096 -> 14336 8.46 against 8.56, 4096 -> 128256 53.5
    // against 55.4, two rows of Q6_K 4096 -> 14336 12.7 against 13.4).  Three and four rows, whose
    // arithmetic per item is longer, keep about MM8S_DEPTH_BYTES worth of items on their way
    // (three rows 4096 -> 6144: 6.6 against 6.9 us with one), fewer when a reused ring is too short.
    // Pairs of Q4_K or Q5_K blocks of a long row (4.5 and 5.5 KiB an item, its 32 pieces a whole row
    // or eight blocks apart) come in late enough for two: 14336 -> 4096 Q4_K 9.1 against 10.1 us,
    // Q5_K 11.0 against 11.5 (Q6_K pairs, 6.6 KiB: 13.6 against 13.3; whole blocks of 24 rows,
    // 4096 -> 6144: 5.46 against 5.41).
    uint32_t depth = pi == 0 ? ((fold && item_bytes < 6144u) ? 2u : 1u)
                             : std::min(gq::MM8S_MAX_DEPTH, std::max(2u, (gq::MM8S_DEPTH_BYTES + item_bytes / 2u) / item_bytes));
    if (ctx->mm8s_depth) depth = std::min(gq::MM8S_MAX_DEPTH, ctx->mm8s_depth);
    while (depth > (split ? 1u : 2u) && slots < items && slots < gq::mm8s_min_slots(depth)) --depth;
    if (slots < items && slots < gq::mm8s_min_slots(depth)) return -1;
    const bool areg = ipt <= 16 && pi <= 1 && ctx->mm8s_areg && !(fold && ctx->call_glu) && !split;
    // Where the other kernels were timed faster (rows of 14336 and of 4096 elements over 4096 to
    // 128256 weight rows): several activation rows of long weight rows, whose preparation every
    // workgroup repeats in full (Q4_K 2 x 14336 -> 4096: 13.0 against 12.2 us); Q6_K other than
    // one long row (14336 -> 4096: 14.6 against 16.3 us, 11008 -> 4096: 11.7 against 14.4) or two
    // short ones (4096 -> 14336: 12.9 against 16.0), the integer-dot GEMV being ahead for one short
    // row (4096 -> 14336: 11.5 against 12.8 us) and the arithmetic of a Q6_K item costing the same
    // for a low tile as for a full one.
    // Five to eight activation rows lead over at most 32 weight rows per CU or rows of at most 8
    // blocks (Q4_K 6 x 4096 -> 6144: 9.9 against 10.2 us, 8 x 2048 -> 14336: 10.6 against 12.0; 6 x
    // 4096 -> 14336: 15.0 against 14.3, 6 x 4096 -> 28672: 24.7 against 21.6), Q6_K over at most 32
    // weight rows per CU (5 x 4096 -> 4096: 11.7 against 12.0; 5 x 2048 -> 14336: 13.6 against 12.9).
    const bool few_rows = n <= static_cast<size_t>(32) * cus;
    if (!ctx->mm8s_all) {
        if (pi == 2 && !(few_rows || (groups <= 8 && kind != MM8_Q6K))) return -1;
        if (mm >= 2 && groups > 16 && !split) return -1;
        // Tiles of fewer than 16 weight rows block by block, the matrix cores mostly idle, lose to
        // the K split of the other form for long rows (Q4_K 8192 -> 2048: 7.6 against 8.6 us) and
        // to the integer-dot GEMV for one row of Q5_K (4096 -> 2048: 4.8-5.2 against 5.6).  In
        // pairs of blocks they lead (8192 -> 2048: Q4_K 5.8 against 7.5, Q5_K 5.8 against 6.8;
        // 14336 -> 2048 Q4_K 7.1 against 9.9; Q5_K 4096 -> 2048 4.5 against 4.7).
        if (!fold && kind != MM8_Q6K && groups > 16 && rows_per_wg < 16) return -1;
        if (!fold && kind == MM8_Q5K && mm == 1 && n < static_cast<size_t>(12) * cus) return -1;
        // Q6_K: one row of 40 blocks and more, in pairs of blocks from 20 (5120 -> 4096: 6.4 against 8.1 us, 6144 -> 4096: 7.3 against
        // 8.7 us for the GEMV, 8192 -> 4096: 9.1 against 10.2; 4096 -> 4096: 6.3 against 6.0), or two short rows
        // three rows of K <= 4096 (4096 -> 14336: 14.7 against 16.6 us), four over at most 32 weight rows per
        // CU or rows of at most 8 blocks (4096 -> 6144: 8.7 against 10.4; 4096 -> 14336: 17.4 against 16.7)
        if (kind == MM8_Q6K && !((mm == 1 && (groups >= 40 || (fold && groups >= 20))) || ((mm == 2 || mm == 3) && areg) ||
                                 (mm == 4 && areg && (few_rows || groups <= 8)) || pi == 2 || split))
            return -1;
        // Q8_0, two rows over at most 8 weight rows per CU: its GEMV stays ahead (4096 -> 1024: 5.9 against 7.1 us)
        if (kind == MM8_Q8_0 && mm == 2 && n <= static_cast<size_t>(8) * cus) return -1;
        // one short row over at most 4 weight rows per CU: the integer-dot GEMV stays ahead
        // (4096 -> 1024: Q4_K 4.6 against 5.0 us, Q5_K 4.9 against 5.0; 8192 -> 1024 Q4_K: 6.3 against 5.9 here)
        if (mm == 1 && rows_per_wg <= 4 && groups <= 16) return -1;
    }
    const uint32_t steps = (((groups + 7u) / 8u + 1u) / 2u) * mm; // preparation steps per wave
    int variant;
    if (areg) variant = pi == 1 ? 2 : (steps <= 1 ? 0 : 1);
    else variant = (pi == 0 && steps > 2) ? 6 : 3 + static_cast<int>(pi);
    hipFunction_t fn = ctx->mm8s[sfmt][variant];
    if (split) {
        if (ctx->call_glu && !glu_vector_ok(ctx)) return kNeedPlainActivations;
        fn = ctx->mm8s_split[sfmt][pi][ctx->call_glu ? 1 : 0];
    } else if (fold) {
        // variants 0, 1 (registers), 3, 6 (LDS) of one activation row
        const int fv = variant <= 1 ? variant : variant == 3 ? 2 : 3;
        if (ctx->call_glu) {
            if (!glu_vector_ok(ctx)) return kNeedPlainActivations;
            fn = ctx->mm8s_fold[sfmt][fv + 2];
        } else {
            fn = ctx->mm8s_fold[sfmt][ctx->call_elem ? fv + 6 : fv];
        }
    } else if (glu) {
        const int gv = variant <= 4 ? variant : variant == 6 ? 5 : -1; // no gated build of p4_e4
        if (gv < 0) return -1;
        fn = ctx->mm8s_gated[sfmt][gv];
    } else if (ctx->call_glu) {
        const int gv = variant == 3 ? 0 : variant == 4 ? 1 : variant == 6 ? 2 : variant == 5 ? 3 : -1; // (the rest keep their planes in registers: rows of at most 4096 elements, not a down projection's)
        if (gv < 0 || !glu_vector_ok(ctx)) return kNeedPlainActivations;
        fn = ctx->mm8s_glu[sfmt][gv];
    } else if (ctx->call_elem) {
        const int ev = variant <= 4 ? variant : variant == 6 ? 5 : -1; // no 16-bit build of p4_e4
        if (ev < 0) return kNeedPlainActivations;
        fn = ctx->mm8s_e16[sfmt][ev];
    }
    Mm8Params P{};
    P.glu = ctx->call_glu;
    P.glu_off = ctx->call_glu_off;
    P.w = w;
    P.w2 = w2;
    P.glu_relu = glu_relu ? 1u : 0u;
    P.x = x;
    P.y = y;
    P.n = static_cast<uint32_t>(n);
    P.k = static_cast<uint32_t>(k);
    P.groups = groups;
    P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
    P.m = mm;
    P.ldx = row_stride_x(ctx, k);
    P.ldy = static_cast<uint32_t>(n);
    P.tiles = tiles;
    P.grid = grid;
    P.act_bf16 = act_bf16 ? 1u : 0u;
    P.elem = ctx->call_elem;
    P.xrows = ctx->identity_rows;
    P.rows_per_wg = rows_per_wg;
    P.tile_rows = tile_rows;
    P.ring_slots = slots;
    P.wg_tiles = wg_tiles;
    P.last_wg_rows = P.n - (grid - 1u) * rows_per_wg;
    P.last_wg_tiles = (P.last_wg_rows + tile_rows - 1u) / tile_rows;
    const gq::Mm8sLds L = gq::mm8s_lds_layout(lds_groups, mm, pairs, item_bytes, slots, subs, glu);
    P.lds_ctrl = L.ctrl;
    P.lds_ring = L.ring;
    P.depth = depth;
    P.progress = ctx->call_seq && ctx->prefetch_announce ? ctx->progress : nullptr;
    P.progress_seq = ctx->call_seq;
    const uint32_t lds = L.total;
    if (split) {
        P.ksplit = ksplit;
        P.kslice_groups = kslice;
        P.part = S->mm8_part;
        P.arrive = S->mm8_arrive;
    }
    return launch(ctx, fn, grid * ksplit, (gq::MM8S_CWAVES + gq::MM8S_LOADERS) * 64, lds, stream, &P, sizeof P, split);
}

// Q4_K, Q5_K and Q6_K on the int8 matrix cores, activation rows in passes of at most 8 (a pass keeps
// its rows' digit planes in LDS and reads the weights once).  Returns -1 when the shape does
// not fit the kernel (LDS for the prepared activations, alignment), so that the caller
// takes the GEMV kernels.
// `w2` != null selects the gated form: `w` holds the n gate rows, `w2` the n up rows, and
// y = act(gate . x) * (up . x) (Q4_K and Q5_K, one pass only).
int run_mm8(gllmq_ctx *ctx, Scratch &S, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n,
            size_t k, bool act_bf16, void *stream, bool one_pass_only = false, const uint8_t *w2 = nullptr,
            bool glu_relu = false)
{
    const int kind = mm8_kind(f.dtype);
    if (!ctx->use_mm8 || kind < 0) return -1;
    const bool glu = w2 != nullptr;
    if (glu && kind != MM8_Q4K && kind != MM8_Q5K) return -1;
    if (glu) one_pass_only = true;
    // The row thresholds below say where the GEMV kernels are as fast; that holds while a GEMV
    // workgroup's prepared activations (848 bytes per row and 256 elements) leave room for
    // several workgroups per CU.  Two rows of more than 9728 elements do not (one workgroup of
    // four waves per CU: 35 against 25 us for Q6_K 14336 -> 4096), so they come here.
    const bool gemv_cramped = 848u * m * ((k + 255) / 256) > 64u * 1024u;
    // One row of 40 blocks and more over few weight rows (a down projection): the K split below
    // gives every CU a slice, and the Q5_K and Q6_K kernels here then beat the GEMV, which walks
    // such a row with three or four waves (11008 -> 4096: Q6_K 15.5 against 17.6 us, Q5_K 13.2
    // against 16.6; 14336 -> 4096: 17.5 against 17.7 and 14.5 against 15.5).
    const bool long_single = m == 1 && (k + 255) / 256 >= 40 && ctx->mm8_ksplit_max > 1 &&
                             ((n + 31) / 32) * 2 <= static_cast<size_t>(ctx->num_cus);
    if (kind == MM8_Q6K && (ctx->mm8_q6k_min_m == 0 || (m < ctx->mm8_q6k_min_m && !gemv_cramped && !long_single))) return -1;
    if (kind == MM8_Q5K && !glu && (ctx->mm8_q5k_min_m == 0 || (m < ctx->mm8_q5k_min_m && !long_single))) return -1;
    if (kind == MM8_Q8_0 && (ctx->mm8_q8_0_min_m == 0 || (m < ctx->mm8_q8_0_min_m && !gemv_cramped))) return -1;
    if (kind == MM8_Q8_0 && k < 256) return -1; // its fetch window is one whole group of 8 blocks
    // One row of Q4_K over at most 4 weight rows per CU: a workgroup's prologue and the meeting of
    // the K slices outweigh what the matrix cores save, the integer-dot GEMV is ahead
    // (4096 -> 1024: 4.5-4.7 against 5.1-5.3 us, 8192 -> 1024: 6.2-6.3 against 7.4, 14336 -> 512: 8.4 against 9.4).
    if (kind == MM8_Q4K && m == 1 && !glu && ctx->mm8_small_to_gemv && n <= static_cast<size_t>(4) * static_cast<size_t>(ctx->num_cus)) return -1;
    if (!aligned(x, 16) || k % 8 != 0) return -1; // the kernel loads activations as aligned vectors
    const uint32_t groups = static_cast<uint32_t>((k + 255) / 256);
    // K split: with tiles for at most half of the CUs, 2..8 workgroups share each tile and take
    // a slice of K each (whole passes of 8 blocks); the slices meet inside the launch.  The
    // meeting costs about 2 us, so a slice keeps at least two passes, unless only a shorter slice
    // lets the prepared activations of all rows fit the LDS (one pass over the weights then beats
    // the alternatives by more than that).
    const uint32_t tiles = static_cast<uint32_t>((n + 31) / 32), ppt_row = (groups + 7u) / 8u;
    auto pairs_for = [](uint32_t rows) { return rows <= 2 ? 1u : (rows <= 4 ? 2u : 4u); };
    const uint32_t m_pass = static_cast<uint32_t>(std::min<size_t>(m, 8));
    uint32_t ksplit = 1, slice_passes = ppt_row;
    if (!glu && ctx->mm8_ksplit_max > 1 && ppt_row >= 2 && (kind != MM8_Q8_0 || k % 256 == 0)) {
        auto fits = [&](uint32_t slices) {
            const uint32_t passes = (ppt_row + slices - 1) / slices;
            return mm8_lds_bytes(std::min(groups, passes * 8u), m_pass, pairs_for(m_pass), kind) <= 160u * 1024u;
        };
        const uint32_t most = std::min(ppt_row, ctx->mm8_ksplit_max);
        uint32_t want = 1;
        if (tiles * 2u <= static_cast<uint32_t>(ctx->num_cus))
            want = std::max(1u, std::min({ static_cast<uint32_t>(ctx->num_cus) / tiles, ppt_row / 2u, most }));
        while (want < most && !fits(want)) ++want;
        // more workgroups than CUs run in rounds: whole rounds beat one and a half
        const uint32_t cus = static_cast<uint32_t>(ctx->num_cus);
        if (want > 1 && want * tiles > cus && tiles <= cus)
            for (uint32_t w2 = want; w2 <= most; ++w2)
                if ((w2 * tiles) % cus == 0) { want = w2; break; }
        if (fits(want)) {
            slice_passes = (ppt_row + want - 1) / want;
            ksplit = (ppt_row + slice_passes - 1) / slice_passes; // every slice gets at least one pass
        }
        if (static_cast<size_t>(ksplit) * m_pass * n > gq::MM8_SPLIT_PART_FLOATS) ksplit = 1;
        if (ksplit == 1) slice_passes = ppt_row;
    }
    const uint32_t lds_groups = ksplit > 1 ? std::min(groups, slice_passes * 8u) : groups;
    // Rows per pass: as many as the prepared activations leave room for in the 160 KiB of LDS.
    uint32_t rows_per_pass = m_pass;
    while (rows_per_pass > 0 && mm8_lds_bytes(lds_groups, rows_per_pass, pairs_for(rows_per_pass), kind) > 160u * 1024u)
        --rows_per_pass;
    if (rows_per_pass == 0) return -1;
    if (one_pass_only && rows_per_pass < m) return -1;
    if (ctx->call_elem) return kNeedPlainActivations; // these kernels read and write f32
    // gated activations (a feed-forward block's down projection): passes of five to eight rows have a kernel for them
    if (ctx->call_glu) {
        const size_t last_pass = m - ((m - 1) / rows_per_pass) * rows_per_pass;
        if (glu || rows_per_pass < 5 || last_pass < 5 || !glu_vector_ok(ctx) || !ctx->mm8_gated_p4[kind]) return kNeedPlainActivations;
    }
    for (size_t m0 = 0; m0 < m; m0 += rows_per_pass) {
        const uint32_t mm = static_cast<uint32_t>(std::min<size_t>(rows_per_pass, m - m0));
        const int pi = mm <= 2 ? 0 : (mm <= 4 ? 1 : 2);
        const uint32_t pairs = 1u << pi;
        const uint32_t lds = mm8_lds_bytes(lds_groups, mm, pairs, kind);
        Mm8Params P{};
        P.ksplit = ksplit;
        P.kslice_groups = slice_passes * 8u;
        P.part = S.mm8_part;
        P.arrive = S.mm8_arrive;
        P.w2 = w2;
        P.glu_relu = glu_relu ? 1u : 0u;
        P.glu = ctx->call_glu;
        P.glu_off = ctx->call_glu_off;
        P.w = w;
        P.x = x + m0 * row_stride_x(ctx, k);
        P.y = y + m0 * n;
        P.n = static_cast<uint32_t>(n);
        P.k = static_cast<uint32_t>(k);
        P.groups = groups;
        P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
        P.m = mm;
        P.ldx = row_stride_x(ctx, k);
        P.ldy = static_cast<uint32_t>(n);
        P.tiles = (P.n + 31u) / 32u;
        P.act_bf16 = act_bf16 ? 1u : 0u;
        P.xrows = ctx->identity_rows;
        // preparation steps per wave: two 256-element blocks per step
        const uint32_t ppt = slice_passes, steps = ((ppt + 1u) / 2u) * mm;
        int ei = steps <= 1 ? 0 : (steps <= 2 ? 1 : 2);
        while (ei < 2 && !ctx->mm8[kind][pi][ei]) ++ei; // not every (pairs, early) pair is built
        const int gi = kind == MM8_Q5K ? 1 : 0;
        uint32_t grid = std::min<uint32_t>(P.tiles, std::max(1u, static_cast<uint32_t>(ctx->num_cus) / ksplit));
        if (ksplit > 1) grid = std::min(grid, gq::MM8_SPLIT_MAX_LISTS);
        P.grid = grid; // workgroups per slice: launch index = tile list * ksplit + slice
        hipFunction_t fn = glu ? ctx->mm8_glu[gi][pi][ei] : ctx->mm8[kind][pi][ei];
        // The register-resident variants are compiled for a fixed number of passes per tile and
        // take a tile's pass from the item's position in the register ring; a last K slice with
        // fewer passes than the others would break that, so such a split runs the LDS variants.
        const bool even_slices = ksplit == 1 || ppt_row % slice_passes == 0;
        if (pi <= 1 && ppt <= 2 && even_slices)
            fn = glu ? ctx->mm8_glu_areg[gi][pi][ei][ppt - 1] : ctx->mm8_areg[kind][pi][ei][ppt - 1];
        if (ctx->call_glu) fn = ctx->mm8_gated_p4[kind]; // (pi == 2: checked above)
        int rc = launch(ctx, fn, grid * ksplit, 512, lds, stream, &P, sizeof P, ksplit > 1);
        if (rc != GLLMQ_OK) return rc;
    }
    return GLLMQ_OK;
}

constexpr uint32_t kMmfMaxRowTiles = 16384;

// Launch shape of the GEMM for one matmul, and the scratch it needs.
struct MmfPlan {
    uint32_t groups, row_tiles, ksplit, bps;
    size_t img_bytes, need;
};

MmfPlan plan_mmf(const gllmq_ctx *ctx, size_t m, size_t n, size_t k)
{
    MmfPlan L{};
    L.groups = static_cast<uint32_t>((k + 255) / 256);
    L.row_tiles = static_cast<uint32_t>((n + 255) / 256);
    uint32_t ksplit = std::max(1u, static_cast<uint32_t>(ctx->num_cus) / std::max(1u, L.row_tiles));
    ksplit = std::min(ksplit, L.groups);
    L.bps = (L.groups + ksplit - 1) / ksplit;
    L.ksplit = (L.groups + L.bps - 1) / L.bps; // every workgroup gets at least one block
    const size_t rows = std::min<size_t>(m, 64);
    // scratch: the activation images of one pass, then the partial sums
    L.img_bytes = static_cast<size_t>(L.groups) * mmf_image_bytes(rows <= 32 ? 1u : 2u);
    L.need = L.img_bytes + (L.ksplit > 1 ? static_cast<size_t>(L.ksplit) * rows * n * 4 : 0);
    return L;
}

int run_mmf(gllmq_ctx *ctx, Scratch &S, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n,
            size_t k, bool act_bf16, void *stream, size_t min_m = 9)
{
    if (!ctx->use_mmf || m < min_m) return -1;
    const int fmt = f.dtype == T_Q8_0 ? 3 : f.dtype == T_Q6_K ? 2 : f.dtype == T_Q5_K ? 1 : 0;
    if (fmt == 3 && k < 256) return -1; // the Q8_0 fetch window is one whole group of 8 blocks
    if (!aligned(x, 16) || k % 4 != 0) return -1; // activation rows are loaded as aligned float4
    if (ctx->call_glu && !glu_vector_ok(ctx)) return kNeedPlainActivations;
    const MmfPlan L = plan_mmf(ctx, m, n, k);
    const uint32_t groups = L.groups, row_tiles = L.row_tiles, ksplit = L.ksplit, bps = L.bps;
    if (row_tiles > kMmfMaxRowTiles) return -1;
    // the GEMM kernels address weight rows with 32-bit byte offsets from the start of the matrix
    if (n * gllmq_row_bytes(f.dtype, k) > 0xFFFFFFFFull) return -1;
    const size_t rows_per_pass = 64, img_bytes = L.img_bytes;
    int grc = grow_scratch(ctx, S, &S.mmf, &S.mmf_bytes, L.need, stream, "quantized_matmul (GEMM)");
    if (grc != GLLMQ_OK) return grc;
    for (size_t m0 = 0; m0 < m; m0 += rows_per_pass) {
        const uint32_t mm = static_cast<uint32_t>(std::min(rows_per_pass, m - m0));
        const uint32_t mt = mm <= 32 ? 1u : 2u;
        MmfParams P{};
        P.w = w;
        P.elem = ctx->call_elem;
        P.ldx = row_stride_x(ctx, k);
        P.x = elem_at(ctx, x, m0 * P.ldx);
        P.y = elem_at(ctx, y, m0 * n);
        P.ximg = static_cast<uint8_t *>(S.mmf);
        P.partial = reinterpret_cast<float *>(static_cast<uint8_t *>(S.mmf) + img_bytes);
        P.n = static_cast<uint32_t>(n);
        P.k = static_cast<uint32_t>(k);
        P.groups = groups;
        P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
        P.m = mm;
        P.ldy = static_cast<uint32_t>(n);
        P.row_tiles = row_tiles;
        P.ksplit = ksplit;
        P.blocks_per_split = bps;
        P.act_bf16 = act_bf16 ? 1u : 0u;
        MmfPrepParams Q{ P.x, P.ximg, mm, P.k, P.ldx, P.act_bf16, P.elem, ctx->call_glu, ctx->call_glu_off };
        int rc = launch2d(ctx, ctx->mmf_prep[mt - 1], groups, 16, 64, 0, stream, &Q, sizeof Q, true);
        if (rc != GLLMQ_OK) return rc;
        rc = launch(ctx, ctx->mmf_q4k[fmt][mt - 1][act_bf16 ? 1 : 0], row_tiles * ksplit, 512, mmf_lds_bytes(mt, fmt), stream,
                    &P, sizeof P, true);
        if (rc == GLLMQ_OK && ksplit > 1) {
            MmfReduceParams R{ P.partial, P.y, mm, P.n, P.ldy, ksplit, P.elem };
            const uint64_t quads = (static_cast<uint64_t>(mm) * n + 3) / 4;
            rc = launch(ctx, ctx->mmf_reduce, static_cast<uint32_t>((quads + 255) / 256), 256, 0, stream, &R, sizeof R, true);
        }
        if (rc != GLLMQ_OK) return rc;
    }
    return GLLMQ_OK;
}

// Launch geometry of the streamed GEMM (mmfs.hip.inc) for one matmul; ok = false when the shape is
// left to the three-launch form.
struct MmfsPlan {
    bool ok = false;
    uint32_t groups = 0, ksplit = 1, rows_per_wg = 0, grid = 0, wg_tiles = 0, tile_rows = 0, slots = 0, depth = 2,
             lds_ctrl = 0, lds_ring = 0, lds = 0;
    size_t img_bytes = 0, need = 0; // scratch: one image per block of K (32 activation rows per launch), then the slice sums
};

MmfsPlan plan_mmfs(const gllmq_ctx *ctx, const Format &f, size_t m, size_t n, size_t k)
{
    MmfsPlan L;
    const int fmt = f.dtype == T_Q5_K ? 1 : f.dtype == T_Q4_K ? 0 : -1;
    if (!ctx->use_mmf || !ctx->use_mmfs || fmt < 0 || m == 0 || n == 0) return L;
    const uint32_t cus = static_cast<uint32_t>(ctx->num_cus);
    if (n < static_cast<size_t>(ctx->mmfs_min_rows) * cus) return L;
    // Timed against the three-launch form at 16 and 32 rows: ahead on matrices of up to 6144 x 4096
    // (32 rows: 13.2 against 22.0 us at 4096 x 4096, 15.5 against 19.2 at 6144 x 4096: two launches
    // instead of three, no pass over partial sums in a launch of its own), behind from 14336 x 4096
    // on (24.6 against 23.9 us; 38.1 against 34.0 at 28672 x 4096; 31.8 against 26.7 at 4096 x 14336):
    // one arithmetic wave per SIMD does not hide its own dependent instructions once the stream
    // is long enough to matter.
    if (!ctx->mmfs_all && n * k > (40ull << 20)) return L;
    L.groups = static_cast<uint32_t>((k + 255) / 256);
    // a workgroup multiplies four blocks of K (one per arithmetic wave); the row ranges are as many
    // as give every CU a workgroup
    L.ksplit = (L.groups + gq::MMFS_CWAVES - 1u) / gq::MMFS_CWAVES;
    const uint32_t ranges = std::max(1u, cus / L.ksplit);
    L.rows_per_wg = static_cast<uint32_t>((n + ranges - 1) / ranges);
    L.grid = static_cast<uint32_t>((n + L.rows_per_wg - 1) / L.rows_per_wg);
    // the loader's 32-bit offsets stay inside a workgroup's rows
    if (static_cast<size_t>(L.rows_per_wg) * gllmq_row_bytes(f.dtype, k) > 0xFFFFFFFFull) return L;
    L.wg_tiles = (L.rows_per_wg + 31u) / 32u;
    L.tile_rows = (L.rows_per_wg + L.wg_tiles - 1u) / L.wg_tiles; // equal heights, <= 32
    if (L.ksplit > 1 && L.grid > kScratchArriveBytes / 4u) return L; // one arrival counter per row range
    const uint32_t pieces = fmt == 1 ? gq::Mm8sFormat<1>::PIECES : gq::Mm8sFormat<0>::PIECES;
    const uint32_t item_bytes = L.tile_rows * pieces * 16u;
    L.lds_ctrl = 0;
    L.lds_ring = (static_cast<uint32_t>(sizeof(gq::Mm8sCtrl)) + gq::MMFS_RED_BUFS * gq::MMFS_CWAVES * 4096u + 1023u) & ~1023u;
    const uint32_t items = L.wg_tiles * gq::MMFS_CWAVES;
    L.slots = std::min(items, (160u * 1024u - L.lds_ring) / item_bytes);
    if (L.slots < items) L.slots -= L.slots % gq::MMFS_LOADERS; // a reused ring is a whole number of rounds of the loaders
    L.depth = ctx->mm8s_depth ? std::min(gq::MM8S_MAX_DEPTH, ctx->mm8s_depth) : 1u; // as for the one-row kernels (12.7 against 12.8 us at 32 x 4096 x 4096, 10.5 against 10.8 at 2048 x 2048)
    while (L.depth > 2u && L.slots < items && L.slots < gq::mm8s_min_slots(L.depth)) --L.depth;
    if (L.slots < items && L.slots < gq::mm8s_min_slots(L.depth)) return L;
    L.lds = L.lds_ring + L.slots * item_bytes;
    L.img_bytes = static_cast<size_t>(L.groups) * gq::MmfLanes::image;
    L.need = L.img_bytes + (L.ksplit > 1 ? static_cast<size_t>(L.ksplit) * L.grid * L.wg_tiles * 4096u : 0u);
    L.ok = true;
    return L;
}

// Q4_K and Q5_K, more than 8 activation rows, from `mmfs_min_rows` weight rows per CU up: the
// streamed GEMM, 32 activation rows per launch (a preparation launch for their images, then the
// GEMM, which leaves y complete).  Returns -1 when the shape is left to run_mmf.
int run_mmfs(gllmq_ctx *ctx, Scratch &S, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n,
             size_t k, bool act_bf16, void *stream, size_t min_m = 9)
{
    if (m < min_m) return -1;
    if (!aligned(x, 16) || k % 4 != 0) return -1; // activation rows are loaded as aligned float4
    const MmfsPlan L = plan_mmfs(ctx, f, m, n, k);
    if (!L.ok) return -1;
    if (ctx->call_glu && !glu_vector_ok(ctx)) return kNeedPlainActivations;
    int grc = grow_scratch(ctx, S, &S.mmf, &S.mmf_bytes, L.need, stream, "quantized_matmul (GEMM)");
    if (grc != GLLMQ_OK) return grc;
    const int fmt = f.dtype == T_Q5_K ? 1 : 0;
    for (size_t m0 = 0; m0 < m; m0 += 32) {
        const uint32_t mm = static_cast<uint32_t>(std::min<size_t>(32, m - m0));
        MmfPrepParams Q{ elem_at(ctx, x, m0 * row_stride_x(ctx, k)), static_cast<uint8_t *>(S.mmf), mm, static_cast<uint32_t>(k),
                         row_stride_x(ctx, k), act_bf16 ? 1u : 0u, ctx->call_elem, ctx->call_glu, ctx->call_glu_off };
        int rc = launch2d(ctx, ctx->mmf_prep_lanes, L.groups, 16, 64, 0, stream, &Q, sizeof Q, true);
        if (rc != GLLMQ_OK) return rc;
        Mm8Params P{};
        P.w = w;
        P.x = static_cast<const float *>(S.mmf); // the images
        P.y = elem_at(ctx, y, m0 * n);
        P.elem = ctx->call_elem;
        P.n = static_cast<uint32_t>(n);
        P.k = static_cast<uint32_t>(k);
        P.groups = L.groups;
        P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
        P.m = mm;
        P.ldx = static_cast<uint32_t>(k);
        P.ldy = static_cast<uint32_t>(n);
        P.grid = L.grid;
        P.ksplit = L.ksplit;
        P.kslice_groups = gq::MMFS_CWAVES;
        P.part = reinterpret_cast<float *>(static_cast<uint8_t *>(S.mmf) + L.img_bytes);
        P.arrive = S.mm8_arrive;
        P.rows_per_wg = L.rows_per_wg;
        P.tile_rows = L.tile_rows;
        P.ring_slots = L.slots;
        P.wg_tiles = L.wg_tiles;
        P.last_wg_rows = P.n - (L.grid - 1u) * L.rows_per_wg;
        P.last_wg_tiles = (P.last_wg_rows + L.tile_rows - 1u) / L.tile_rows;
        P.lds_ctrl = L.lds_ctrl;
        P.lds_ring = L.lds_ring;
        P.depth = L.depth;
        rc = launch(ctx, ctx->mmfs[fmt][act_bf16 ? 1 : 0], L.grid * L.ksplit, (gq::MMFS_CWAVES + gq::MMFS_LOADERS) * 64, L.lds,
                    stream, &P, sizeof P, true);
        if (rc != GLLMQ_OK) return rc;
    }
    return GLLMQ_OK;
}

// Q4_K and Q5_K, 9 to 16 rows of f32 activations, from `mmfr_min_rows` weight rows per CU up: the
// streamed GEMM whose arithmetic waves prepare their own activations (mmfr.hip.inc), one launch and
// nothing else.  A workgroup multiplies a slice of K of eight blocks (a block per arithmetic wave);
// the slices of a row range meet through the scratch.  Returns -1 for what it does not take.
int run_mmfr(gllmq_ctx *ctx, Scratch &S, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n,
             size_t k, bool act_bf16, void *stream, size_t min_m = 9)
{
    const int fmt = f.dtype == T_Q5_K ? 1 : f.dtype == T_Q4_K ? 0 : -1;
    // (17 rows and more: two ways of sharing a block between two waves were built and timed slower than the three-launch form)
    if (!ctx->use_mmf || !ctx->use_mmfr || fmt < 0 || m < min_m || m > 16 || n == 0) return -1;
    if (act_bf16 || ctx->call_elem || ctx->call_glu) return -1; // plain f32 activations and outputs
    const uint32_t ldx = row_stride_x(ctx, k);
    if (!aligned(x, 16) || k % 4 != 0 || ldx % 4 != 0) return -1; // activation rows are loaded as aligned float4
    const uint32_t cus = static_cast<uint32_t>(ctx->num_cus);
    if (n < static_cast<size_t>(ctx->mmfr_min_rows) * cus) return -1;
    const uint32_t groups = static_cast<uint32_t>((k + 255) / 256);
    const uint32_t pieces = fmt == 1 ? gq::Mm8sFormat<1>::PIECES : gq::Mm8sFormat<0>::PIECES;
    const uint32_t sb = gq::MMFR_CWAVES; // blocks of a slice
    const uint32_t ksplit = (groups + sb - 1u) / sb;
    const uint32_t ranges = std::max(1u, cus / ksplit);
    const uint32_t rows_per_wg = static_cast<uint32_t>((n + ranges - 1) / ranges);
    const uint32_t grid = static_cast<uint32_t>((n + rows_per_wg - 1) / rows_per_wg);
    // the loader's 32-bit offsets stay inside a workgroup's rows
    if (static_cast<size_t>(rows_per_wg) * gllmq_row_bytes(f.dtype, k) > 0xFFFFFFFFull) return -1;
    const uint32_t wg_tiles = (rows_per_wg + 31u) / 32u;
    const uint32_t tile_rows = (rows_per_wg + wg_tiles - 1u) / wg_tiles; // equal heights, <= 32
    if (ksplit > 1 && grid > kScratchArriveBytes / 4u) return -1;       // one arrival counter per row range
    const uint32_t item_bytes = tile_rows * pieces * 16u;
    const uint32_t lds_ring = (static_cast<uint32_t>(sizeof(gq::Mm8sCtrl)) + gq::MMFR_RED_BUFS * gq::MMFR_CWAVES * gq::MMFR_RED_WAVE + 1023u) & ~1023u;
    const uint32_t items = wg_tiles * sb;
    uint32_t slots = std::min(items, (160u * 1024u - lds_ring) / item_bytes);
    if (slots < items) slots -= slots % gq::MMFR_LOADERS; // a reused ring is a whole number of rounds of the loaders
    uint32_t depth = ctx->mm8s_depth ? std::min(gq::MM8S_MAX_DEPTH, ctx->mm8s_depth) : 1u;
    while (depth > 2u && slots < items && slots < gq::mm8s_min_slots(depth)) --depth;
    // (the waves of a tile's blocks run side by side: a ring shorter than two tiles' items would let a loader wait for a wave that waits for it)
    if (slots < items && (slots < gq::mm8s_min_slots(depth) || slots < 2u * sb)) return -1;
    const size_t part_bytes = ksplit > 1 ? static_cast<size_t>(ksplit) * grid * wg_tiles * 2048u : 0u;
    if (part_bytes) {
        int grc = grow_scratch(ctx, S, &S.mmf, &S.mmf_bytes, part_bytes, stream, "quantized_matmul (GEMM)");
        if (grc != GLLMQ_OK) return grc;
    }
    Mm8Params P{};
    P.w = w;
    P.x = x;
    P.y = y;
    P.n = static_cast<uint32_t>(n);
    P.k = static_cast<uint32_t>(k);
    P.groups = groups;
    P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
    P.m = static_cast<uint32_t>(m);
    P.ldx = ldx;
    P.ldy = static_cast<uint32_t>(n);
    P.grid = grid;
    P.ksplit = ksplit;
    P.kslice_groups = sb;
    P.part = static_cast<float *>(S.mmf);
    P.arrive = S.mm8_arrive;
    P.rows_per_wg = rows_per_wg;
    P.tile_rows = tile_rows;
    P.ring_slots = slots;
    P.wg_tiles = wg_tiles;
    P.last_wg_rows = P.n - (grid - 1u) * rows_per_wg;
    P.last_wg_tiles = (P.last_wg_rows + tile_rows - 1u) / tile_rows;
    P.lds_ctrl = 0;
    P.lds_ring = lds_ring;
    P.depth = depth;
    return launch(ctx, ctx->mmfr[fmt], grid * ksplit, (gq::MMFR_CWAVES + gq::MMFR_LOADERS) * 64, lds_ring + slots * item_bytes, stream, &P,
                  sizeof P, ksplit > 1);
}

// A chain of batch entries for one launch of mm8c.hip.inc: consecutive matmuls of one format
// (Q4_K or Q5_K), one K <= 4096 and one activation row count <= 2 that the streamed kernels
// would take one by one.  chain_length() says how many entries from `descs` on form one (0 or 1:
// none); run_chain() launches it.
bool chain_entry_ok(const gllmq_ctx *ctx, const gllmq_matmul_desc &d, const gllmq_matmul_desc &first)
{
    const Format *f = find_format(d.ggml_dtype);
    if (!f || (f->dtype != T_Q4_K && f->dtype != T_Q5_K && f->dtype != T_Q8_0)) return false;
    if (f->dtype == T_Q5_K && ctx->mm8_q5k_min_m == 0) return false;
    if (f->dtype == T_Q8_0 && (ctx->mm8_q8_0_min_m == 0 || !ctx->mm8s_q8_0 || d.k % 256 != 0)) return false; // whole groups of 8 blocks
    if (d.ggml_dtype != first.ggml_dtype || d.m != first.m || d.k != first.k) return false;
    if (d.m == 0 || d.m > 2 || d.k == 0 || d.k % 8 != 0 || (d.k + 255) / 256 > 16 || d.n > 0x7FFFFFFFu) return false;
    if (!d.w_dev || !d.x_dev || !d.y_dev || !aligned(d.x_dev, 16) || !aligned(d.y_dev, 4) || !aligned(d.w_dev, f->w_align)) return false;
    const size_t rb = gllmq_row_bytes(d.ggml_dtype, d.k);
    if (rb % f->w_align != 0 || d.w_bytes < d.n * rb) return false;
    const size_t cus = static_cast<size_t>(ctx->num_cus);
    return d.n > 0 && (d.n + cus - 1) / cus >= ctx->chain_min_rows; // rows of the largest share
}

// Whether [a, a + an) and [b, b + bn) share a byte.
bool ranges_meet(const void *a, size_t an, const void *b, size_t bn)
{
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + bn && b0 < a0 + an;
}

constexpr size_t kChainBoxPairs = size_t(1) << 19; // 64-bit words of the mailbox (4 MiB per stream that runs such chains)

// Whether entry `d`, flagged as starting after `prev`, reads (part of) prev's output and nothing
// else, so that it can take its activations from what prev posts: one activation row anywhere
// inside prev's output row, or all rows of an output whose rows are exactly as long as d's.
bool chain_reads_previous(const gllmq_matmul_desc &d, const gllmq_matmul_desc &prev)
{
    const uintptr_t x = reinterpret_cast<uintptr_t>(d.x_dev), y = reinterpret_cast<uintptr_t>(prev.y_dev);
    if (x < y || (x - y) % 4 != 0) return false;
    const size_t at = (x - y) / 4;
    if (d.m == 1) return at + d.k <= prev.n; // (the chain's entries share m)
    return at == 0 && d.k == prev.n;
}

size_t chain_length(const gllmq_ctx *ctx, const gllmq_matmul_desc *descs, size_t count)
{
    if (!ctx->use_chain || !ctx->use_mm8 || !ctx->use_mm8s || count < 2) return 0;
    size_t len = 0, posted = 0; // entries so far, and the mailbox places their posting entries take
    while (len < count && len < gq::MM8C_MAX_ENTRIES && !(descs[len].flags & ~1u) && chain_entry_ok(ctx, descs[len], descs[0])) {
        const gllmq_matmul_desc &d = descs[len];
        const size_t xb = d.m * d.k * 4, yb = d.m * d.n * 4;
        const bool reads_prev = len > 0 && (d.flags & 1u) && ctx->chain_dependent && chain_reads_previous(d, descs[len - 1]) &&
                                posted + descs[len - 1].m * descs[len - 1].n <= kChainBoxPairs;
        // An entry that starts after the one before it and does not simply read its output begins a
        // launch of its own: the launch boundary is the one wait that covers every case.
        if (len > 0 && (d.flags & 1u) && !reads_prev) break;
        // Workgroups run through the entries at their own pace: nothing an entry writes may be
        // anything another entry of the launch reads from memory or writes.
        bool clash = false;
        for (size_t j = 0; j < len && !clash; ++j) {
            const gllmq_matmul_desc &o = descs[j];
            const bool o_reads_prev = j > 0 && (o.flags & 1u); // (then it reads the mailbox, not memory)
            clash = ranges_meet(d.y_dev, yb, o.y_dev, o.m * o.n * 4) || (!o_reads_prev && ranges_meet(d.y_dev, yb, o.x_dev, o.m * o.k * 4)) ||
                    (!reads_prev && ranges_meet(d.x_dev, xb, o.y_dev, o.m * o.n * 4));
        }
        if (clash || ranges_meet(d.y_dev, yb, d.x_dev, xb)) break;
        if (reads_prev) posted += descs[len - 1].m * descs[len - 1].n;
        ++len;
    }
    return len;
}

int run_chain(gllmq_ctx *ctx, Scratch &S, const gllmq_matmul_desc *descs, size_t len, void *stream)
{
    const Format &f = *find_format(descs[0].ggml_dtype);
    const int fmt = f.dtype == T_Q8_0 ? 2 : f.dtype == T_Q5_K ? 1 : 0;
    const uint32_t cus = static_cast<uint32_t>(ctx->num_cus);
    const size_t k = descs[0].k;
    Mm8ChainParams P{};
    P.count = static_cast<uint32_t>(len);
    P.k = static_cast<uint32_t>(k);
    P.groups = static_cast<uint32_t>((k + 255) / 256);
    P.row_bytes = static_cast<uint32_t>(gllmq_row_bytes(f.dtype, k));
    P.m = static_cast<uint32_t>(descs[0].m);
    P.ldx = P.k;
    P.act_bf16 = 0;
    const uint32_t pieces = fmt == 2 ? gq::Mm8sFormat<3>::PIECES : fmt == 1 ? gq::Mm8sFormat<1>::PIECES : gq::Mm8sFormat<0>::PIECES;
    P.slot_bytes = 32u * pieces * 16u; // a slot holds an item of any entry: 32 rows of one block
    // LDS: the preparation's planes, sums and scales; the counters; the partial sums; the ring
    const gq::Mm8Lds prep = gq::mm8_lds_layout(P.groups, P.m, 1u, fmt == 2 ? 0u : 8u, 0u);
    P.lds_ctrl = (prep.red + 15u) & ~15u;
    const uint32_t red = P.lds_ctrl + static_cast<uint32_t>(sizeof(gq::Mm8sCtrl)) + gq::MM8C_MAX_SLOTS * 4u;
    P.lds_ring = (red + gq::MM8C_RED_BUFS * gq::MM8C_CWAVES * 64u * 4u + 1023u) & ~1023u;
    P.depth = ctx->mm8s_depth ? std::min(gq::MM8S_MAX_DEPTH, ctx->mm8s_depth) : 0u; // 0: by the entry's items, see the loader
    if (P.lds_ring >= 160u * 1024u) return -1;
    uint32_t slots = std::min(gq::MM8C_MAX_SLOTS, (160u * 1024u - P.lds_ring) / P.slot_bytes);
    slots -= slots % gq::MM8C_LOADERS;
    if (slots < gq::mm8s_min_slots(std::max(2u, P.depth))) return -1;
    P.ring_slots = slots;
    P.spin_limit = ctx->chain_spin_limit;
    P.epoch0 = ctx->chain_epoch;
    P.error = ctx->chain_error;
    P.progress = ctx->call_seq ? ctx->progress : nullptr;
    P.progress_seq = ctx->call_seq;
    uint32_t launched = 0, box_used = 0;
    for (size_t i = 0; i < len; ++i) {
        const gllmq_matmul_desc &d = descs[i];
        Mm8ChainEntry &E = P.e[i];
        E.w = static_cast<const uint8_t *>(d.w_dev);
        E.x = static_cast<const float *>(d.x_dev);
        E.y = static_cast<float *>(d.y_dev);
        E.n = static_cast<uint32_t>(d.n);
        E.ldy = E.n;
        E.rows_per_wg = (E.n + cus - 1u) / cus;
        E.grid = (E.n + E.rows_per_wg - 1u) / E.rows_per_wg;
        E.wg_tiles = (E.rows_per_wg + 31u) / 32u;
        E.tile_rows = (E.rows_per_wg + E.wg_tiles - 1u) / E.wg_tiles;
        E.last_wg_rows = E.n - (E.grid - 1u) * E.rows_per_wg;
        E.last_wg_tiles = (E.last_wg_rows + E.tile_rows - 1u) / E.tile_rows;
        E.flags = i > 0 ? (d.flags & 1u) : 0u; // the chain's first entry is ordered by the stream
        if (i > 0 && E.flags) { // (chain_length() has checked that it reads the output of the entry before and that the places fit)
            Mm8ChainEntry &B = P.e[i - 1];
            B.flags |= 2u;
            B.box_at = box_used;
            box_used += P.m * B.n;
            E.x_at = B.box_at + static_cast<uint32_t>((static_cast<const float *>(d.x_dev) - static_cast<const float *>(descs[i - 1].y_dev)));
            E.x_ld = B.n;
        }
        // one activation row over tiles of at most 16 weight rows: in pairs of blocks, as run_mm8s() would
        if (ctx->mm8s_fold_on && P.m == 1 && E.tile_rows <= 16 && P.groups > 8) E.flags |= 4u;
        launched = std::max(launched, E.grid);
    }
    bool waits = false, folds = false;
    for (size_t i = 0; i < len; ++i) {
        waits = waits || (P.e[i].flags & 3u) != 0u;
        folds = folds || (P.e[i].flags & 4u) != 0u;
    }
    if (waits) {
        if (box_used > kChainBoxPairs) return -1;
        if (!S.box) {
            // first chain of this kind on the stream: the mailbox, all zero (epochs start at 1).  Not
            // during a capture and not from a block of fixed size: the entries then take a launch each.
            if (S.fixed || stream_is_capturing(stream)) return -1;
            GLLMQ_HIP(ctx, hipSetDevice(ctx->device));
            GLLMQ_HIP(ctx, hipMalloc(&S.box, kChainBoxPairs * 8));
            GLLMQ_HIP(ctx, hipMemset(S.box, 0, kChainBoxPairs * 8));
        }
        P.box = static_cast<unsigned long long *>(S.box);
        ctx->chain_epoch += static_cast<uint32_t>(len);
    }
    P.launched = launched;
    return launch(ctx, ctx->mm8c[fmt][folds ? 1 : 0][waits ? 1 : 0], launched, (gq::MM8C_CWAVES + gq::MM8C_LOADERS) * 64, P.lds_ring + slots * P.slot_bytes,
                  stream, &P, sizeof P, true);
}

int run_gemv(gllmq_ctx *ctx, const Format &f, const uint8_t *w, const float *x, float *y, size_t m, size_t n,
             size_t k, bool act_bf16, void *stream)
{
    const size_t rb = gllmq_row_bytes(f.dtype, k);
    constexpr size_t kChunk = 16384; // elements of K one launch covers (four waves of 4096)
    if (ctx->call_glu && ctx->gemv_f32) return kNeedPlainActivations;
    const uint32_t ldx = row_stride_x(ctx, k);
    // 16-bit elements are read as aligned vectors only
    if (ctx->call_elem && !(aligned(x, 16) && k % 64 == 0 && ldx % 8 == 0)) return kNeedPlainActivations;
    for (size_t m0 = 0; m0 < m; m0 += 2) {
        const uint32_t mm = static_cast<uint32_t>(std::min<size_t>(2, m - m0));
        for (size_t k0 = 0; k0 < k; k0 += kChunk) {
            const size_t kk = std::min(kChunk, k - k0);
            int rc = launch_gemv(ctx, f, w + (k0 / 256) * f.group_bytes, rb, elem_at(ctx, x, m0 * ldx + k0), elem_at(ctx, y, m0 * n), mm,
                                 static_cast<uint32_t>(n), static_cast<uint32_t>(kk), ldx,
                                 static_cast<uint32_t>(n), k0 != 0, act_bf16, stream);
            if (rc != GLLMQ_OK) return rc;
        }
    }
    return GLLMQ_OK;
}

// One quantized matmul on validated arguments: the kernel family by format, rows and shape.
int dispatch_matmul(gllmq_ctx *ctx, Scratch &S, const Format &f, const uint8_t *w, const float *x, float *y, size_t m,
                    size_t n, size_t k, bool bf16, void *stream)
{
    int rc = run_mmfr(ctx, S, f, w, x, y, m, n, k, bf16, stream);
    if (rc >= 0) return rc;
    rc = run_mmfs(ctx, S, f, w, x, y, m, n, k, bf16, stream);
    if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    rc = run_mmf(ctx, S, f, w, x, y, m, n, k, bf16, stream);
    if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    // up to 8 rows: the int8 kernels when one pass over the weights does it, else the GEMM
    rc = run_mm8s(ctx, f, w, x, y, m, n, k, bf16, stream, nullptr, false, &S);
    if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    rc = run_mm8(ctx, S, f, w, x, y, m, n, k, bf16, stream, true);
    if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    if (ctx->mmf_small_min_m > 0) {
        rc = run_mmf(ctx, S, f, w, x, y, m, n, k, bf16, stream, ctx->mmf_small_min_m);
        if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    }
    rc = run_mm8(ctx, S, f, w, x, y, m, n, k, bf16, stream);
    if (rc >= 0 || rc == kNeedPlainActivations) return rc;
    return run_gemv(ctx, f, w, x, y, m, n, k, bf16, stream);
}

size_t ffn_h_bytes(size_t m, size_t ffn) { return ((m * ffn * sizeof(float)) + 255) & ~size_t(255); }
size_t ffn_scratch_bytes(size_t m, size_t ffn) { return ffn_h_bytes(m, ffn) + m * 2 * ffn * sizeof(float); }

// Which kernel the dispatch gives a matmul: the dispatch itself, run with launches and allocations
// switched off (ctx->probe), so that the answer cannot drift from what a call does.  `fn` is the
// kernel when the call is exactly one launch, else null; `launches` counts them.
struct DispatchChoice {
    hipFunction_t fn = nullptr;
    uint32_t launches = 0;
};

template <class Call>
DispatchChoice dispatch_choice(gllmq_ctx *ctx, Call &&call)
{
    ctx->probe = true;
    ctx->probe_launches = 0;
    ctx->probe_fn = nullptr;
    const int rc = call();
    ctx->probe = false;
    DispatchChoice c;
    c.launches = rc == GLLMQ_OK ? ctx->probe_launches : 0u;
    c.fn = c.launches == 1u ? ctx->probe_fn : nullptr;
    return c;
}

// One validated quantized matmul with the scratch of `S` (call_mutex held).
int matmul_on_scratch(gllmq_ctx *ctx, Scratch &S, const void *w, size_t w_bytes, const float *x, float *y, uint32_t dtype,
                      size_t m, size_t n, size_t k, int act_mode, void *stream)
{
    const Format *f = find_format(dtype);
    int rc = check_matmul_args(ctx, f, w, w_bytes, x, y, dtype, m, n, k);
    if (rc >= 0) return rc;
    if (act_mode != GLLMQ_ACT_F32_SPLIT && act_mode != GLLMQ_ACT_BF16)
        return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul: unknown activation mode %d", act_mode);
    const bool bf16 = act_mode == GLLMQ_ACT_BF16;
    if (bf16 && ctx->gemv_f32)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED, "quantized_matmul: bf16 activations are not built for the f32 GEMV flavour");
    return dispatch_matmul(ctx, S, *f, static_cast<const uint8_t *>(w), x, y, m, n, k, bf16, stream);
}

} // namespace

extern "C" {

const char *gllmq_version(void) { return "gllm_hip_quant 0.1 (gfx950)"; }

const char *gllmq_status_string(int status)
{
    switch (status) {
    case GLLMQ_OK: return "ok";
    case GLLMQ_ERR_UNIMPLEMENTED: return "unimplemented";
    case GLLMQ_ERR_BAD_SHAPE: return "bad shape";
    case GLLMQ_ERR_BAD_ALIGNMENT: return "bad alignment";
    case GLLMQ_ERR_HIP: return "hip error";
    case GLLMQ_ERR_INVALID: return "invalid argument";
    default: return "unknown status";
    }
}

size_t gllmq_block_size(uint32_t dtype)
{
    const Format *f = find_format(dtype);
    return f ? f->block_size : 0;
}

size_t gllmq_block_bytes(uint32_t dtype)
{
    const Format *f = find_format(dtype);
    return f ? f->block_bytes : 0;
}

size_t gllmq_row_bytes(uint32_t dtype, size_t k)
{
    const Format *f = find_format(dtype);
    return f ? (k + f->block_size - 1) / f->block_size * f->block_bytes : 0;
}

int gllmq_init(gllmq_ctx **out, int device)
{
    if (!out) return GLLMQ_ERR_INVALID;
    *out = nullptr;
    gllmq_ctx *ctx = new gllmq_ctx;
    ctx->device = device;
    hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) e = hipFree(nullptr); // force context creation
    if (e != hipSuccess) {
        fprintf(stderr, "gllmq_init: device %d: %s\n", device, hipGetErrorString(e));
        delete ctx;
        return GLLMQ_ERR_HIP;
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) == hipSuccess) {
        ctx->num_cus = prop.multiProcessorCount;
        if (strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
            fprintf(stderr, "gllmq_init: device %d is %s; this library holds gfx950 code only\n", device,
                    prop.gcnArchName);
            delete ctx;
            return GLLMQ_ERR_UNIMPLEMENTED;
        }
    }
    const unsigned char *const images[9] = { gllmq_co_codec, gllmq_co_mm8, gllmq_co_mm8s, gllmq_co_mm8s_q8_0, gllmq_co_mm8c,
                                             gllmq_co_mm8_q6k_q8_0, gllmq_co_mmf, gllmq_co_mmfs, gllmq_co_moe };
    for (int i = 0; i < 9; ++i) {
        e = hipModuleLoadData(&ctx->modules[i], images[i]);
        if (e != hipSuccess) {
            fprintf(stderr, "gllmq_init: hipModuleLoadData: %s\n", hipGetErrorString(e));
            for (hipModule_t mod : ctx->modules)
                if (mod) (void)hipModuleUnload(mod);
            delete ctx;
            return GLLMQ_ERR_HIP;
        }
    }
    int rc = GLLMQ_OK;
    char name[64];
    for (int i = 0; i < kNumFormats && rc == GLLMQ_OK; ++i) {
        snprintf(name, sizeof name, "gq_dequant_%s_v1", kFormats[i].tag);
        rc = get_function(ctx, &ctx->dequant[i][0], name);
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_dequant_%s_v4", kFormats[i].tag);
        rc = get_function(ctx, &ctx->dequant[i][1], name);
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_gather_%s_v1", kFormats[i].tag);
        rc = get_function(ctx, &ctx->gather[i][0], name);
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_gather_%s_v4", kFormats[i].tag);
        rc = get_function(ctx, &ctx->gather[i][1], name);
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_gather_%s_e16_v1", kFormats[i].tag);
        rc = get_function(ctx, &ctx->gather_e16[i][0], name);
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_gather_%s_e16_v4", kFormats[i].tag);
        rc = get_function(ctx, &ctx->gather_e16[i][1], name);
        for (int m = 1; m <= 2 && rc == GLLMQ_OK; ++m) {
            snprintf(name, sizeof name, "gq_gemv_%s_m%d", kFormats[i].tag, m);
            rc = get_function(ctx, &ctx->gemv[i][m - 1], name);
            if (rc != GLLMQ_OK) break;
            snprintf(name, sizeof name, "gq_gemv_i8_%s_m%d", kFormats[i].tag, m);
            rc = get_function(ctx, &ctx->gemv_i8[i][m - 1], name);
            if (rc != GLLMQ_OK) break;
            snprintf(name, sizeof name, "gq_gemv_i8_%s_m%d_glu", kFormats[i].tag, m);
            rc = get_function(ctx, &ctx->gemv_i8_glu[i][m - 1], name);
            if (rc != GLLMQ_OK) break;
            snprintf(name, sizeof name, "gq_gemv_i8_%s_m%d_e16", kFormats[i].tag, m);
            rc = get_function(ctx, &ctx->gemv_i8_e16[i][m - 1], name);
        }
        if (rc != GLLMQ_OK) break;
        snprintf(name, sizeof name, "gq_gemv_i8_%s_m1_argmax", kFormats[i].tag);
        rc = get_function(ctx, &ctx->gemv_i8_argmax[i], name);
    }
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_route, "gq_moe_route");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->convert_elem, "gq_convert_elem");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmf_prep[0], "gq_mmf_prep_t1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmf_prep[1], "gq_mmf_prep_t2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmf_prep_lanes, "gq_mmf_prep_lanes");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmf_reduce, "gq_mmf_reduce");
    for (int q = 0; q < 4 && rc == GLLMQ_OK; ++q)
        for (int t = 0; t < 2 && rc == GLLMQ_OK; ++t)
            for (int b = 0; b < 2 && rc == GLLMQ_OK; ++b) {
                snprintf(name, sizeof name, "gq_mmf_%s_t%d%s", q == 3 ? "q8_0" : q == 2 ? "q6k" : q == 1 ? "q5k" : "q4k", t + 1, b ? "_bf16" : "");
                rc = get_function(ctx, &ctx->mmf_q4k[q][t][b], name);
            }
    static const char *const kMm8c[3][2] = { { "gq_mm8c_q4k", "gq_mm8c_q4k_f" }, { "gq_mm8c_q5k", "gq_mm8c_q5k_f" }, { "gq_mm8c_q8_0", "gq_mm8c_q8_0_f" } };
    for (int q = 0; q < 3 && rc == GLLMQ_OK; ++q)
        for (int v = 0; v < 2 && rc == GLLMQ_OK; ++v)
            for (int d = 0; d < 2 && rc == GLLMQ_OK; ++d) {
                snprintf(name, sizeof name, "%s%s", kMm8c[q][v], d ? "_d" : "");
                rc = get_function(ctx, &ctx->mm8c[q][v][d], name);
            }
    for (int q = 0; q < 2 && rc == GLLMQ_OK; ++q)
        for (int b = 0; b < 2 && rc == GLLMQ_OK; ++b) {
            snprintf(name, sizeof name, "gq_mmfs_%s%s", q ? "q5k" : "q4k", b ? "_bf16" : "");
            rc = get_function(ctx, &ctx->mmfs[q][b], name);
        }
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmfr[0], "gq_mmfr_q4k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mmfr[1], "gq_mmfr_q5k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_plan, "gq_moe_plan");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_act, "gq_moe_act");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_combine, "gq_moe_combine");
    for (int i = 0; i < kNumFormats && rc == GLLMQ_OK; ++i) {
        snprintf(name, sizeof name, "gq_moe_gemv_%s", kFormats[i].tag);
        rc = get_function(ctx, &ctx->moe_gemv[i], name);
    }
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[0][0], "gq_moe_mm8_q4k_a1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[0][1], "gq_moe_mm8_q4k_a2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[1][0], "gq_moe_mm8_q6k_a1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[1][1], "gq_moe_mm8_q6k_a2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[2][0], "gq_moe_mm8_q5k_a1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_fn[2][1], "gq_moe_mm8_q5k_a2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_q6k_rows, "gq_moe_mm8_q6k_rows");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8s_fn[MM8_Q4K][0], "gq_moe_mm8s_q4k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8s_fn[MM8_Q5K][0], "gq_moe_mm8s_q5k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8s_fn[MM8_Q6K][0], "gq_moe_mm8s_q6k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8s_fn[MM8_Q4K][1], "gq_moe_mm8s_glu_q4k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8s_fn[MM8_Q5K][1], "gq_moe_mm8s_glu_q5k");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_glu_fn[MM8_Q4K][0], "gq_moe_mm8_glu_q4k_a1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_glu_fn[MM8_Q4K][1], "gq_moe_mm8_glu_q4k_a2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_glu_fn[MM8_Q5K][0], "gq_moe_mm8_glu_q5k_a1");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->moe_mm8_glu_fn[MM8_Q5K][1], "gq_moe_mm8_glu_q5k_a2");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->dequant_wave, "gq_dequant_q4k_wave");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->dequant_wave_q5k, "gq_dequant_q5k_wave");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->argmax_part, "gq_argmax_part");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->argmax_final, "gq_argmax_final");
    if (rc == GLLMQ_OK) {
        static const uint32_t kRows[8] = { 0, 1, 2, 3, 4, 5, 6, 7 };
        hipError_t he = hipMalloc(reinterpret_cast<void **>(&ctx->identity_rows), sizeof kRows);
        if (he == hipSuccess) he = hipMemcpy(ctx->identity_rows, kRows, sizeof kRows, hipMemcpyHostToDevice);
        if (he != hipSuccess) rc = fail(ctx, GLLMQ_ERR_HIP, "row table: %s", hipGetErrorString(he));
    }
    if (rc == GLLMQ_OK) {
        hipError_t he = hipHostMalloc(reinterpret_cast<void **>(&ctx->chain_error), sizeof(uint32_t), hipHostMallocDefault);
        if (he == hipSuccess) *ctx->chain_error = 0u;
        else rc = fail(ctx, GLLMQ_ERR_HIP, "error word: %s", hipGetErrorString(he));
    }
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->touch, "gq_touch");
    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->finish_elem, "gq_finish_elem");
    if (rc == GLLMQ_OK) {
        hipError_t he = hipMalloc(reinterpret_cast<void **>(&ctx->progress), 256);
        if (he == hipSuccess) he = hipMemset(ctx->progress, 0, 256);
        if (he == hipSuccess) he = hipStreamCreateWithFlags(&ctx->side_stream, hipStreamNonBlocking);
        if (he == hipSuccess) he = hipEventCreateWithFlags(&ctx->side_event, hipEventDisableTiming);
        if (he != hipSuccess) rc = fail(ctx, GLLMQ_ERR_HIP, "prefetch stream: %s", hipGetErrorString(he));
    }
    {
        static const struct { int pi, ei; const char *tag; } kMm8[] = {
            { 0, 0, "p1_e1" }, { 0, 1, "p1_e2" }, { 0, 2, "p1_e4" }, { 1, 1, "p2_e2" }, { 1, 2, "p2_e4" }, { 2, 2, "p4_e4" },
        };
        static const char *const kMm8Format[MM8_KINDS] = { "q4k", "q6k", "q5k", "q8_0" };
        for (int q = 0; q < MM8_KINDS; ++q)
            for (const auto &k : kMm8) {
                snprintf(name, sizeof name, "gq_mm8_%s_%s", kMm8Format[q], k.tag);
                if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mm8[q][k.pi][k.ei], name);
                for (int a = 1; a <= 2 && k.pi <= 1 && rc == GLLMQ_OK; ++a) {
                    snprintf(name, sizeof name, "gq_mm8_%s_%s_a%d", kMm8Format[q], k.tag, a);
                    rc = get_function(ctx, &ctx->mm8_areg[q][k.pi][k.ei][a - 1], name);
                }
                if (k.pi == 2) {
                    snprintf(name, sizeof name, "gq_mm8_%s_%s_g", kMm8Format[q], k.tag);
                    if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mm8_gated_p4[q], name);
                }
                if (q != MM8_Q4K && q != MM8_Q5K) continue;
                const int gi = q == MM8_Q5K ? 1 : 0;
                snprintf(name, sizeof name, "gq_mm8_glu_%s_%s", kMm8Format[q], k.tag);
                if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->mm8_glu[gi][k.pi][k.ei], name);
                for (int a = 1; a <= 2 && k.pi <= 1 && rc == GLLMQ_OK; ++a) {
                    snprintf(name, sizeof name, "gq_mm8_glu_%s_%s_a%d", kMm8Format[q], k.tag, a);
                    rc = get_function(ctx, &ctx->mm8_glu_areg[gi][k.pi][k.ei][a - 1], name);
                }
            }
        if (rc == GLLMQ_OK) rc = get_function(ctx, &ctx->glu_act, "gq_glu_act");
        static const char *const kMm8sFormat[4] = { "q4k", "q5k", "q6k", "q8_0" };
        static const char *const kMm8s[7] = { "p1_e1_a", "p1_e2_a", "p2_e4_a", "p1_e2", "p2_e4", "p4_e4", "p1_e4" };
        for (int q = 0; q < 4; ++q)
            for (int v = 0; v < 7 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_%s", kMm8sFormat[q], kMm8s[v]);
                rc = get_function(ctx, &ctx->mm8s[q][v], name);
            }
        static const char *const kMm8sGated[6] = { "p1_e1_a", "p1_e2_a", "p2_e4_a", "p1_e2", "p2_e4", "p1_e4" };
        for (int q = 0; q < 2; ++q)
            for (int v = 0; v < 6 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_%s_glu", q ? "q5k" : "q4k", kMm8sGated[v]);
                rc = get_function(ctx, &ctx->mm8s_gated[q][v], name);
            }
        static const char *const kMm8sE16[6] = { "p1_e1_a", "p1_e2_a", "p2_e4_a", "p1_e2", "p2_e4", "p1_e4" };
        for (int q = 0; q < 4; ++q)
            for (int v = 0; v < 6 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_%s_e16", kMm8sFormat[q], kMm8sE16[v]);
                rc = get_function(ctx, &ctx->mm8s_e16[q][v], name);
            }
        static const char *const kMm8sFold[10] = { "p1_e1_a_f", "p1_e2_a_f", "p1_e2_f", "p1_e4_f", "p1_e2_g_f", "p1_e4_g_f",
                                                   "p1_e1_a_f_e16", "p1_e2_a_f_e16", "p1_e2_f_e16", "p1_e4_f_e16" };
        for (int q = 0; q < 4; ++q)
            for (int v = 0; v < 10 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_%s", kMm8sFormat[q], kMm8sFold[v]);
                rc = get_function(ctx, &ctx->mm8s_fold[q][v], name);
            }
        for (int q = 0; q < 4; ++q)
            for (int v = 0; v < 4 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_p%d_e4%s_s", kMm8sFormat[q], 1 + (v & 1), (v & 2) ? "_g" : "");
                rc = get_function(ctx, &ctx->mm8s_split[q][v & 1][v >> 1], name);
            }
        static const char *const kMm8sGlu[4] = { "p1_e2_g", "p2_e4_g", "p1_e4_g", "p4_e4_g" };
        for (int q = 0; q < 4; ++q)
            for (int v = 0; v < 4 && rc == GLLMQ_OK; ++v) {
                snprintf(name, sizeof name, "gq_mm8s_%s_%s", kMm8sFormat[q], kMm8sGlu[v]);
                rc = get_function(ctx, &ctx->mm8s_glu[q][v], name);
            }
    }
    if (rc == GLLMQ_OK) {
        // the kernels that say when they start (the streamed forms and their chain)
        auto add = [&](hipFunction_t f) { if (f) ctx->announces.insert(f); };
        for (auto &q : ctx->mm8s) for (hipFunction_t f : q) add(f);
        for (auto &q : ctx->mm8s_gated) for (hipFunction_t f : q) add(f);
        for (auto &q : ctx->mm8s_e16) for (hipFunction_t f : q) add(f);
        for (auto &q : ctx->mm8s_glu) for (hipFunction_t f : q) add(f);
        for (auto &q : ctx->mm8s_fold) for (hipFunction_t f : q) add(f);
        for (auto &q : ctx->mm8s_split) for (auto &r : q) for (hipFunction_t f : r) add(f);
        for (auto &q : ctx->mm8c) for (auto &v : q) for (hipFunction_t f : v) add(f);
    }
    // the scratch array of the entry point that allocates nothing: found (and thereby placed on
    // this device) now, while allocating is allowed
    if (rc == GLLMQ_OK) rc = gq_noalloc_init(ctx, device);
    if (rc != GLLMQ_OK) {
        fprintf(stderr, "gllmq_init: %s\n", ctx->err.c_str());
        for (hipModule_t mod : ctx->modules)
            if (mod) (void)hipModuleUnload(mod);
        delete ctx;
        return rc;
    }
    ctx->gemv_waves = static_cast<uint32_t>(ctx->num_cus) * 8u;
    *out = ctx;
    return GLLMQ_OK;
}

void gllmq_destroy(gllmq_ctx *ctx)
{
    if (!ctx) return;
    for (Scratch &S : ctx->scratch) free_scratch(S);
    for (CachedWeights &W : ctx->weights)
        if (W.dev) (void)hipFree(W.dev);
    if (ctx->identity_rows) (void)hipFree(ctx->identity_rows);
    if (ctx->chain_error) (void)hipHostFree(ctx->chain_error);
    if (ctx->side_stream) {
        (void)hipStreamSynchronize(ctx->side_stream);
        (void)hipStreamDestroy(ctx->side_stream);
    }
    if (ctx->side_event) (void)hipEventDestroy(ctx->side_event);
    if (ctx->progress) (void)hipFree(ctx->progress);
    for (hipModule_t mod : ctx->modules)
        if (mod) (void)hipModuleUnload(mod);
    delete ctx;
}

const char *gllmq_last_error(const gllmq_ctx *ctx)
{
    if (!ctx) return "NULL context";
    // a copy per calling thread: another thread's failing call may replace the context's string
    static thread_local std::string copy;
    {
        std::lock_guard<std::mutex> g(const_cast<gllmq_ctx *>(ctx)->err_mutex);
        copy = ctx->err;
    }
    return copy.c_str();
}

int gllmq_set_option(gllmq_ctx *ctx, const char *name, long value)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    if (!name) return fail(ctx, GLLMQ_ERR_INVALID, "set_option: NULL name");
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const std::string n(name);
    const uint32_t u = static_cast<uint32_t>(std::max(0l, value));
    if (n == "gemv_f32") ctx->gemv_f32 = value != 0;
    else if (n == "mm8") ctx->use_mm8 = value != 0;
    else if (n == "mmf") ctx->use_mmf = value != 0;
    else if (n == "mm8s") ctx->use_mm8s = value != 0;
    else if (n == "mmfs") ctx->use_mmfs = value != 0;
    else if (n == "mmfr") ctx->use_mmfr = value != 0;
    else if (n == "mmfr_min_rows") ctx->mmfr_min_rows = std::max(1u, u);
    else if (n == "chain") ctx->use_chain = value != 0;
    else if (n == "chain_dependent") ctx->chain_dependent = value != 0;
    else if (n == "chain_spin_limit") ctx->chain_spin_limit = u;
    else if (n == "chain_min_rows") ctx->chain_min_rows = std::max(1u, u);
    else if (n == "lm_head_fused") ctx->lm_head_fused = value != 0;
    else if (n == "elem_fused") ctx->elem_fused = value != 0;
    else if (n == "ffn_glu_load") ctx->ffn_glu_load = value != 0;
    else if (n == "ffn_streamed") ctx->ffn_streamed = value != 0;
    else if (n == "mmfs_all") ctx->mmfs_all = value != 0;
    else if (n == "mmfs_min_rows") ctx->mmfs_min_rows = std::max(1u, u);
    else if (n == "batch_overlap") ctx->batch_overlap = value != 0;
    else if (n == "mm8s_all") ctx->mm8s_all = value != 0;
    else if (n == "mm8s_depth") ctx->mm8s_depth = u;
    else if (n == "mm8s_areg") ctx->mm8s_areg = value != 0;
    else if (n == "mm8s_fold") ctx->mm8s_fold_on = value != 0;
    else if (n == "mm8s_split") ctx->mm8s_split_on = value != 0;
    else if (n == "mm8s_q8_0") ctx->mm8s_q8_0 = value != 0;
    else if (n == "mm8_small_to_gemv") ctx->mm8_small_to_gemv = value != 0;
    else if (n == "mm8s_min_rows") ctx->mm8s_min_rows = std::max(1u, u);
    else if (n == "ffn_fused") ctx->ffn_fused = value != 0;
    else if (n == "mmf_small_min_m") ctx->mmf_small_min_m = u;
    else if (n == "mm8_ksplit") ctx->mm8_ksplit_max = u;
    else if (n == "mm8_q6k_min_m") ctx->mm8_q6k_min_m = u;
    else if (n == "mm8_q5k_min_m") ctx->mm8_q5k_min_m = u;
    else if (n == "mm8_q8_0_min_m") ctx->mm8_q8_0_min_m = u;
    else if (n == "moe_mm8") ctx->moe_mm8 = value != 0;
    else if (n == "moe_mm8_q6k") ctx->moe_mm8_q6k = value != 0;
    else if (n == "moe_mm8_rows") ctx->moe_mm8_rows = value != 0;
    else if (n == "moe_glu") ctx->moe_glu = value != 0;
    else if (n == "moe_streamed") ctx->moe_streamed = u;
    else if (n == "moe_depth") ctx->moe_depth = u;
    else if (n == "moe_slices") ctx->moe_slices = u;
    else if (n == "prefetch") ctx->prefetch = value != 0;
    else if (n == "prefetch_wgs") ctx->prefetch_wgs = u;
    else if (n == "prefetch_threads") ctx->prefetch_threads = std::min(256u, std::max(64u, u & ~63u));
    else if (n == "prefetch_timeout_us") ctx->prefetch_timeout_us = u;
    else if (n == "prefetch_flags") ctx->prefetch_flags = u;
    else if (n == "prefetch_announce") ctx->prefetch_announce = value != 0;
    else if (n == "prefetch_min_kib") ctx->prefetch_min_kib = u;
    else if (n == "weights_cache_mib") ctx->weights_cache_limit = static_cast<size_t>(u) << 20;
    else return fail(ctx, GLLMQ_ERR_INVALID, "set_option: unknown option %s", name);
    return GLLMQ_OK;
}

const char *gllmq_last_kernel_name(const gllmq_ctx *ctx)
{
    if (!ctx || !ctx->last_kernel) return "";
    const auto it = ctx->kernel_names.find(ctx->last_kernel);
    return it == ctx->kernel_names.end() ? "" : it->second.c_str();
}

int gllmq_dequantize(gllmq_ctx *ctx, const void *blocks, size_t n_bytes, float *out, size_t n_out,
                     uint32_t dtype, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *f = find_format(dtype);
    if (!f)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "dequantize: ggml dtype %u is not covered (supported: Q8_0=8, Q4_K=12, Q5_K=13, Q6_K=14)", dtype);
    const size_t nb = std::min(n_bytes / f->block_bytes, n_out / f->block_size);
    if (nb == 0) return GLLMQ_OK;
    if (!blocks || !out) return fail(ctx, GLLMQ_ERR_INVALID, "dequantize: NULL device pointer");
    if (!aligned(out, 4)) return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "dequantize: output must be 4-byte aligned");
    uint64_t n_quads = static_cast<uint64_t>(nb) * (f->block_size / 4);
    const int vec = aligned(out, 16) ? 1 : 0;
    const uint64_t want = (n_quads + 255) / 256;
    const uint32_t grid = static_cast<uint32_t>(std::min<uint64_t>(want, static_cast<uint64_t>(ctx->num_cus) * 64));
    struct { const void *b; float *o; uint64_t n; } args = { blocks, out, n_quads };
    hipFunction_t fn = ctx->dequant[format_index(dtype)][vec];
    if (vec && aligned(blocks, 16) && dtype == T_Q4_K) fn = ctx->dequant_wave;
    if (vec && aligned(blocks, 16) && dtype == T_Q5_K) fn = ctx->dequant_wave_q5k;
    return launch(ctx, fn, grid, 256, 0, stream, &args, sizeof args);
}

int gllmq_quant_gather(gllmq_ctx *ctx, const void *table, size_t table_bytes, uint32_t dtype, size_t vocab,
                       size_t hidden, const uint32_t *ids, size_t count, float scale, float *out, void *stream)
{
    return gllmq_quant_gather_elem(ctx, table, table_bytes, dtype, vocab, hidden, ids, count, scale, out, GLLMQ_ELEM_F32, stream);
}

int gllmq_quant_gather_elem(gllmq_ctx *ctx, const void *table, size_t table_bytes, uint32_t dtype, size_t vocab,
                            size_t hidden, const uint32_t *ids, size_t count, float scale, void *out, int elem, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    if (elem != GLLMQ_ELEM_F32 && elem != GLLMQ_ELEM_F16 && elem != GLLMQ_ELEM_BF16)
        return fail(ctx, GLLMQ_ERR_INVALID, "quant_gather: unknown element type %d", elem);
    const bool e16 = elem != GLLMQ_ELEM_F32;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *f = find_format(dtype);
    if (!f)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "quant_gather: ggml dtype %u is not covered (supported: Q8_0=8, Q4_K=12, Q5_K=13, Q6_K=14)", dtype);
    if (count == 0 || hidden == 0) return GLLMQ_OK;
    if (!table || !ids || !out) return fail(ctx, GLLMQ_ERR_INVALID, "quant_gather: NULL device pointer");
    if (hidden % 4 != 0) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quant_gather: hidden = %zu is not a multiple of 4", hidden);
    if (vocab > 0xFFFFFFFFu || hidden > 0x7FFFFFFFu || count > 0x7FFFFFFFu)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quant_gather: dimension exceeds its 32-bit range");
    const size_t rb = gllmq_row_bytes(dtype, hidden);
    if (table_bytes < vocab * rb)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quant_gather: table has %zu bytes, %zu rows of %zu elements need %zu",
                    table_bytes, vocab, hidden, vocab * rb);
    if (!aligned(ids, 4) || !aligned(out, e16 ? 2 : 4))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "quant_gather: ids must be 4-byte aligned, the output aligned to its element");
    GatherParams P{};
    P.table = static_cast<const uint8_t *>(table);
    P.ids = ids;
    P.out = static_cast<float *>(out);
    P.vocab = static_cast<uint32_t>(vocab);
    P.hidden = static_cast<uint32_t>(hidden);
    P.row_bytes = static_cast<uint32_t>(rb);
    P.quads_per_row = static_cast<uint32_t>(hidden / 4);
    P.count = static_cast<uint32_t>(count);
    P.scale = scale;
    P.elem = static_cast<uint32_t>(elem);
    const int vec = aligned(out, e16 ? 8 : 16) ? 1 : 0; // hidden is a multiple of 4, so every row then is
    // (a one-block-per-wave form as in gq_dequant_q4k_wave measured the same: 15.9 against 16.0 us)
    return launch2d(ctx, (e16 ? ctx->gather_e16 : ctx->gather)[format_index(dtype)][vec], (P.quads_per_row + 255u) / 256u,
                    static_cast<uint32_t>(std::min<size_t>(count, 65535)), 256, 0, stream, &P, sizeof P);
}

int gllmq_argmax(gllmq_ctx *ctx, const float *logits, size_t rows, size_t n, size_t ld, uint32_t *token, float *value,
                 void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (rows == 0) return GLLMQ_OK;
    if ((!logits && n > 0) || !token) return fail(ctx, GLLMQ_ERR_INVALID, "argmax: NULL device pointer");
    if (n > 0xFFFFFFFEu || ld > 0xFFFFFFFFu || rows > 0x7FFFFFFFu || ld < n)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "argmax: n = %zu, ld = %zu, rows = %zu out of range", n, ld, rows);
    if (!aligned(logits, 4) || !aligned(token, 4) || (value && !aligned(value, 4)))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "argmax: buffers must be 4-byte aligned");
    Scratch *S = nullptr;
    int src = acquire_scratch(ctx, stream, &S);
    if (src != GLLMQ_OK) return src;
    ArgmaxParams P{};
    P.keys = S->argmax_keys;
    P.n = static_cast<uint32_t>(n);
    P.ld = static_cast<uint32_t>(ld);
    P.parts = static_cast<uint32_t>(std::min<size_t>(gq::ARGMAX_MAX_PARTS, std::max<size_t>(1, (n + 4095) / 4096)));
    P.chunk = static_cast<uint32_t>((n + P.parts - 1) / P.parts);
    for (size_t r0 = 0; r0 < rows; r0 += gq::ARGMAX_MAX_ROWS) {
        const uint32_t rr = static_cast<uint32_t>(std::min<size_t>(gq::ARGMAX_MAX_ROWS, rows - r0));
        P.logits = logits + r0 * ld;
        P.token = token + r0;
        P.value = value ? value + r0 : nullptr;
        int rc = launch2d(ctx, ctx->argmax_part, P.parts, rr, 256, 0, stream, &P, sizeof P);
        if (rc == GLLMQ_OK && P.parts > 1) rc = launch(ctx, ctx->argmax_final, rr, 256, 0, stream, &P, sizeof P);
        if (rc != GLLMQ_OK) return rc;
    }
    return GLLMQ_OK;
}

int gllmq_lm_head_argmax(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x, uint32_t dtype, size_t n, size_t k,
                         float *logits, uint32_t *token, float *value, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (!token) return fail(ctx, GLLMQ_ERR_INVALID, "lm_head_argmax: NULL token pointer");
    if (!aligned(token, 4) || (value && !aligned(value, 4)))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "lm_head_argmax: buffers must be 4-byte aligned");
    if (n == 0) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "lm_head_argmax: n = 0");
    const Format *f = find_format(dtype);
    // checked as the one-row matmul it is; without a logits buffer the activations stand in for it
    int rc = check_matmul_args(ctx, f, w, w_bytes, x, logits ? logits : const_cast<float *>(x), dtype, 1, n, k);
    if (rc >= 0) return rc;
    Scratch *S = nullptr;
    rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    // The matvec whose workgroups leave their best candidate behind: the one-row GEMV of Q6_K and
    // Q8_0 (the types of GGUF output matrices) where one launch covers K; the workgroup that
    // finishes last picks among the candidates.  With a logits buffer it runs where the GEMV is
    // the kernel gllmq_quantized_matmul gives the shape anyway (dispatch_choice() asks the dispatch
    // itself), so that the logits are that call's bit for bit; without one, always.
    const size_t rb = gllmq_row_bytes(dtype, k);
    const bool gemv_type = dtype == 14u || dtype == 8u;
    bool gemv_anyway = true;
    if (ctx->lm_head_fused && gemv_type && !ctx->gemv_f32 && k <= 16384 && logits) {
        const DispatchChoice c = dispatch_choice(ctx, [&] {
            return dispatch_matmul(ctx, *S, *f, static_cast<const uint8_t *>(w), x, logits, 1, n, k, false, stream);
        });
        gemv_anyway = c.fn != nullptr && c.fn == ctx->gemv_i8[format_index(dtype)][0];
    }
    if (ctx->lm_head_fused && gemv_type && !ctx->gemv_f32 && k <= 16384 && gemv_anyway) {
        GemvPlan L = plan_gemv(ctx, 1, static_cast<uint32_t>(n), static_cast<uint32_t>(k), rb, ctx->gemv_waves);
        if (L.grid <= gq::ARGMAX_MAX_PARTS * gq::ARGMAX_MAX_ROWS) {
            GemvParams &P = L.P;
            P.w = static_cast<const uint8_t *>(w);
            P.x = x;
            P.y = logits;
            P.ldx = static_cast<uint32_t>(k);
            P.ldy = static_cast<uint32_t>(n);
            P.x_vec = aligned(x, 16);
            P.keys = S->argmax_keys;
            P.ticket = S->mm8_arrive + kLmHeadTicketAt;
            P.token = token;
            P.value = value;
            return launch(ctx, ctx->gemv_i8_argmax[format_index(dtype)], L.grid, L.threads, L.lds, stream, &P, sizeof P, true);
        }
    }
    if (!logits)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "lm_head_argmax: this matrix (ggml dtype %u, k = %zu) goes through the matmul and the token choice one "
                    "after the other, which needs a logits buffer of n floats", dtype, k);
    rc = dispatch_matmul(ctx, *S, *f, static_cast<const uint8_t *>(w), x, logits, 1, n, k, false, stream);
    if (rc != GLLMQ_OK) return rc;
    return gllmq_argmax(ctx, logits, 1, n, n, token, value, stream);
}

int gllmq_quantized_matmul_ex(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x, float *y,
                              uint32_t dtype, size_t m, size_t n, size_t k, int act_mode, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    return matmul_on_scratch(ctx, *S, w, w_bytes, x, y, dtype, m, n, k, act_mode, stream);
}

namespace {

int convert_elems(gllmq_ctx *ctx, const void *src, void *dst, size_t count, uint32_t elem, bool widen, void *stream)
{
    gq::ConvertParams C{};
    C.src = src;
    C.dst = dst;
    C.count = count;
    C.elem = elem;
    C.widen = widen ? 1u : 0u;
    const uint32_t grid = static_cast<uint32_t>(std::min<size_t>((count + 255) / 256, 4096));
    return launch(ctx, ctx->convert_elem, std::max(1u, grid), 256, 0, stream, &C, sizeof C, true);
}

size_t elem_scratch_bytes(size_t m, size_t n, size_t k) { return ((m * k * 4 + 255) & ~size_t(255)) + m * n * 4; }

// Whether the kernels convert 16-bit elements in their own loads and stores: all but the GEMV when
// it covers K in several launches (which add up in y), and its f32 flavour.
bool elem_in_kernel(const gllmq_ctx *ctx, size_t m, size_t k)
{
    (void)m;
    return ctx->elem_fused && !ctx->gemv_f32 && k <= 16384;
}

} // namespace

namespace {

// One validated quantized matmul over 16-bit activations and outputs with the scratch of `S`
// (call_mutex held); elem is GLLMQ_ELEM_F16 or GLLMQ_ELEM_BF16.
int matmul_elem_on_scratch(gllmq_ctx *ctx, Scratch &S, const void *w, size_t w_bytes, const void *x, void *y, uint32_t dtype,
                           size_t m, size_t n, size_t k, int elem, void *stream)
{
    const Format *f = find_format(dtype);
    int rc = check_matmul_args(ctx, f, w, w_bytes, static_cast<const float *>(x), static_cast<float *>(y), dtype, m, n, k);
    if (rc >= 0) return rc;
    if (elem_in_kernel(ctx, m, k)) {
        ctx->call_elem = static_cast<uint32_t>(elem);
        rc = dispatch_matmul(ctx, S, *f, static_cast<const uint8_t *>(w), static_cast<const float *>(x),
                             static_cast<float *>(y), m, n, k, false, stream);
        ctx->call_elem = 0;
        if (rc != kNeedPlainActivations) return rc; // else: the kernel for this shape reads f32 only
    }
    rc = grow_scratch(ctx, S, &S.elem, &S.elem_bytes, elem_scratch_bytes(m, n, k), stream, "quantized_matmul_elem");
    if (rc != GLLMQ_OK) return rc;
    float *xf = static_cast<float *>(S.elem);
    float *yf = reinterpret_cast<float *>(static_cast<uint8_t *>(S.elem) + ((m * k * 4 + 255) & ~size_t(255)));
    rc = convert_elems(ctx, x, xf, m * k, static_cast<uint32_t>(elem), true, stream);
    if (rc == GLLMQ_OK) rc = dispatch_matmul(ctx, S, *f, static_cast<const uint8_t *>(w), xf, yf, m, n, k, false, stream);
    if (rc == GLLMQ_OK) rc = convert_elems(ctx, yf, y, m * n, static_cast<uint32_t>(elem), false, stream);
    return rc;
}

} // namespace

int gllmq_quantized_matmul_elem(gllmq_ctx *ctx, const void *w, size_t w_bytes, const void *x, void *y, uint32_t dtype,
                                size_t m, size_t n, size_t k, int elem, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (elem == GLLMQ_ELEM_F32)
        return gllmq_quantized_matmul_ex(ctx, w, w_bytes, static_cast<const float *>(x), static_cast<float *>(y), dtype, m, n,
                                         k, GLLMQ_ACT_F32_SPLIT, stream);
    if (elem != GLLMQ_ELEM_F16 && elem != GLLMQ_ELEM_BF16)
        return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_elem: unknown element type %d", elem);
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    return matmul_elem_on_scratch(ctx, *S, w, w_bytes, x, y, dtype, m, n, k, elem, stream);
}

int gllmq_reserve_matmul_elem(gllmq_ctx *ctx, uint32_t dtype, size_t m, size_t n, size_t k, int elem, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    int rc = gllmq_reserve_matmul(ctx, dtype, m, n, k, stream);
    // (which kernel takes the shape also depends on the pointers' alignment: room for the widened copies either way)
    if (rc != GLLMQ_OK || elem == GLLMQ_ELEM_F32 || m == 0 || n == 0 || k == 0) return rc;
    Scratch *S = nullptr;
    rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    return grow_scratch(ctx, *S, &S->elem, &S->elem_bytes, elem_scratch_bytes(m, n, k), stream, "reserve_matmul_elem");
}

int gllmq_ffn_swiglu(gllmq_ctx *ctx, const void *gate_w, const void *up_w, size_t gate_up_bytes_each, uint32_t dtype_gate_up,
                     const void *down_w, size_t down_bytes, uint32_t dtype_down, const float *x, float *out, size_t m,
                     size_t hidden, size_t ffn, int relu_gate, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *fg = find_format(dtype_gate_up), *fd = find_format(dtype_down);
    if (!fg || !fd)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "ffn_swiglu: ggml dtype %u / %u is not covered (supported: Q8_0=8, Q4_K=12, Q5_K=13, Q6_K=14)",
                    dtype_gate_up, dtype_down);
    if (m == 0 || hidden == 0) return GLLMQ_OK;
    if (ffn == 0) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "ffn_swiglu: ffn = 0");
    if (!up_w) return fail(ctx, GLLMQ_ERR_INVALID, "ffn_swiglu: NULL device pointer");
    // the three matrices are checked as the matmuls they are (the intermediate buffers stand in
    // for the activations that are not the caller's)
    int rc = check_matmul_args(ctx, fg, gate_w, gate_up_bytes_each, x, out, dtype_gate_up, m, ffn, hidden);
    if (rc >= 0) return rc;
    rc = check_matmul_args(ctx, fg, up_w, gate_up_bytes_each, x, out, dtype_gate_up, m, ffn, hidden);
    if (rc >= 0) return rc;
    rc = check_matmul_args(ctx, fd, down_w, down_bytes, x, out, dtype_down, m, hidden, ffn);
    if (rc >= 0) return rc;
    if (ffn > 0x7FFFFFFFu / 2u) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "ffn_swiglu: ffn exceeds 2^30-1");

    // scratch: h [m][ffn], then gate/up results [m][2 ffn] for the form with three steps
    const size_t h_bytes = ffn_h_bytes(m, ffn);
    const size_t need = ffn_scratch_bytes(m, ffn);
    Scratch *Sp = nullptr;
    rc = acquire_scratch(ctx, stream, &Sp);
    if (rc != GLLMQ_OK) return rc;
    Scratch &S = *Sp;
    rc = grow_scratch(ctx, S, &S.ffn, &S.ffn_bytes, need, stream, "ffn_swiglu");
    if (rc != GLLMQ_OK) return rc;
    float *h = static_cast<float *>(S.ffn);
    float *gu = reinterpret_cast<float *>(static_cast<uint8_t *>(S.ffn) + h_bytes);
    const uint8_t *gw = static_cast<const uint8_t *>(gate_w), *uw = static_cast<const uint8_t *>(up_w);

    // gate and up in one launch with the activation in its epilogue (Q4_K / Q5_K, up to 8 rows)
    rc = -1;
    if (ctx->ffn_fused && ctx->ffn_streamed && m <= 4) rc = run_mm8s(ctx, *fg, gw, x, h, m, ffn, hidden, false, stream, uw, relu_gate != 0);
    if (rc < 0 && ctx->ffn_fused && m <= 8) rc = run_mm8(ctx, S, *fg, gw, x, h, m, ffn, hidden, false, stream, true, uw, relu_gate != 0);
    if (rc > 0) return rc;
    if (rc < 0) {
        // three steps: the two products (one matmul when the up rows follow the gate rows in
        // memory), the activation, the down projection
        const size_t rb = gllmq_row_bytes(dtype_gate_up, hidden);
        const bool stacked = uw == gw + ffn * rb;
        gq::GluActParams A{};
        A.h = h;
        A.m = static_cast<uint32_t>(m);
        A.ffn = static_cast<uint32_t>(ffn);
        A.relu_gate = relu_gate ? 1u : 0u;
        if (stacked) {
            rc = dispatch_matmul(ctx, S, *fg, gw, x, gu, m, 2 * ffn, hidden, false, stream);
            A.g = gu;
            A.u = gu + ffn;
            A.ld = static_cast<uint32_t>(2 * ffn);
        } else {
            rc = dispatch_matmul(ctx, S, *fg, gw, x, gu, m, ffn, hidden, false, stream);
            if (rc == GLLMQ_OK) rc = dispatch_matmul(ctx, S, *fg, uw, x, gu + m * ffn, m, ffn, hidden, false, stream);
            A.g = gu;
            A.u = gu + m * ffn;
            A.ld = static_cast<uint32_t>(ffn);
        }
        if (rc != GLLMQ_OK) return rc;
        // the down projection reads act(gate) * up straight from the two results where its kernel
        // can; else the activation runs as a launch of its own and writes h
        const size_t up_off = static_cast<size_t>(A.u - A.g);
        if (ctx->ffn_glu_load && up_off <= 0xFFFFFFFFu) {
            ctx->call_glu = relu_gate ? 2u : 1u;
            ctx->call_glu_off = static_cast<uint32_t>(up_off);
            ctx->call_ldx = A.ld;
            rc = dispatch_matmul(ctx, S, *fd, static_cast<const uint8_t *>(down_w), gu, out, m, hidden, ffn, false, stream);
            ctx->call_glu = ctx->call_glu_off = ctx->call_ldx = 0;
            if (rc != kNeedPlainActivations) return rc;
        }
        rc = launch2d(ctx, ctx->glu_act, static_cast<uint32_t>((ffn + 255) / 256),
                      static_cast<uint32_t>(std::min<size_t>(m, 65535)), 256, 0, stream, &A, sizeof A);
        if (rc != GLLMQ_OK) return rc;
    }
    return dispatch_matmul(ctx, S, *fd, static_cast<const uint8_t *>(down_w), h, out, m, hidden, ffn, false, stream);
}

namespace {

// What the element-type forms of the feed-forward block and of the expert matvec have in common:
// activations of a 16-bit type are widened into the stream's scratch (exact), the f32 entry point
// runs on them, and unless the result can go straight to `out` (f32, nothing to add) it goes to
// scratch too and one small launch writes out = round(result) or out = round(out + result).
struct ElemStage {
    const float *x = nullptr; // what the f32 entry point reads
    float *result = nullptr;  // where it writes
    bool finish = false;
};

int elem_stage_begin(gllmq_ctx *ctx, const void *x, void *out, size_t count, int elem, int flags, void *stream, const char *what,
                     ElemStage *st)
{
    if (elem != GLLMQ_ELEM_F32 && elem != GLLMQ_ELEM_F16 && elem != GLLMQ_ELEM_BF16)
        return fail(ctx, GLLMQ_ERR_INVALID, "%s: unknown element type %d", what, elem);
    if (flags & ~GLLMQ_OUT_ACCUMULATE) return fail(ctx, GLLMQ_ERR_INVALID, "%s: unknown flag bits 0x%x", what, flags);
    st->x = static_cast<const float *>(x);
    st->result = static_cast<float *>(out);
    st->finish = elem != GLLMQ_ELEM_F32 || (flags & GLLMQ_OUT_ACCUMULATE);
    if (!st->finish || count == 0) return GLLMQ_OK;
    if (!x || !out) return fail(ctx, GLLMQ_ERR_INVALID, "%s: NULL device pointer", what);
    if (!aligned(x, 2) || !aligned(out, 2)) return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "%s: x and out must be aligned to their element", what);
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    const size_t each = (count * 4 + 255) & ~size_t(255);
    rc = grow_scratch(ctx, *S, &S->elem, &S->elem_bytes, 2 * each, stream, what);
    if (rc != GLLMQ_OK) return rc;
    st->result = reinterpret_cast<float *>(static_cast<uint8_t *>(S->elem) + each);
    if (elem != GLLMQ_ELEM_F32) {
        float *xf = static_cast<float *>(S->elem);
        rc = convert_elems(ctx, x, xf, count, static_cast<uint32_t>(elem), true, stream);
        st->x = xf;
    }
    return rc;
}

int elem_stage_end(gllmq_ctx *ctx, const ElemStage &st, void *out, size_t count, int elem, int flags, void *stream)
{
    if (!st.finish || count == 0) return GLLMQ_OK;
    gq::ConvertParams C{};
    C.src = st.result;
    C.dst = out;
    C.count = count;
    C.elem = static_cast<uint32_t>(elem);
    C.accumulate = (flags & GLLMQ_OUT_ACCUMULATE) ? 1u : 0u;
    const uint32_t grid = static_cast<uint32_t>(std::min<size_t>((count + 255) / 256, 4096));
    return launch(ctx, ctx->finish_elem, std::max(1u, grid), 256, 0, stream, &C, sizeof C, true);
}

} // namespace

int gllmq_ffn_swiglu_elem(gllmq_ctx *ctx, const void *gate_w, const void *up_w, size_t gate_up_bytes_each, uint32_t dtype_gate_up,
                          const void *down_w, size_t down_bytes, uint32_t dtype_down, const void *x, void *out, size_t m,
                          size_t hidden, size_t ffn, int relu_gate, int elem, int flags, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    ElemStage st;
    int rc = elem_stage_begin(ctx, x, out, m * hidden, elem, flags, stream, "ffn_swiglu", &st);
    if (rc != GLLMQ_OK) return rc;
    rc = gllmq_ffn_swiglu(ctx, gate_w, up_w, gate_up_bytes_each, dtype_gate_up, down_w, down_bytes, dtype_down, st.x, st.result, m,
                          hidden, ffn, relu_gate, stream);
    if (rc != GLLMQ_OK) return rc;
    return elem_stage_end(ctx, st, out, m * hidden, elem, flags, stream);
}

int gllmq_moe_matvec_elem(gllmq_ctx *ctx, const void *gate, size_t gate_bytes, size_t gate_expert_stride, const void *up,
                          size_t up_bytes, size_t up_expert_stride, uint32_t dtype_gu, const void *down, size_t down_bytes,
                          size_t down_expert_stride, uint32_t dtype_dn, const void *x, void *out, size_t tokens, size_t hidden,
                          size_t ffn, size_t experts, size_t top_k, const uint32_t *route_expert, const float *route_weight,
                          const uint32_t *route_len, int relu_gate, int elem, int flags, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    ElemStage st;
    int rc = elem_stage_begin(ctx, x, out, tokens * hidden, elem, flags, stream, "moe_matvec", &st);
    if (rc != GLLMQ_OK) return rc;
    rc = gllmq_moe_matvec(ctx, gate, gate_bytes, gate_expert_stride, up, up_bytes, up_expert_stride, dtype_gu, down, down_bytes,
                          down_expert_stride, dtype_dn, st.x, st.result, tokens, hidden, ffn, experts, top_k, route_expert,
                          route_weight, route_len, relu_gate, stream);
    if (rc != GLLMQ_OK) return rc;
    return elem_stage_end(ctx, st, out, tokens * hidden, elem, flags, stream);
}

int gllmq_quantized_matmul(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x, float *y,
                           uint32_t dtype, size_t m, size_t n, size_t k, void *stream)
{
    return gllmq_quantized_matmul_ex(ctx, w, w_bytes, x, y, dtype, m, n, k, GLLMQ_ACT_F32_SPLIT, stream);
}

namespace {

// One launch (or chained launch) of a batch, as gllmq_quantized_matmul_batch will enqueue it.
struct BatchUnit {
    size_t first, len;
    bool ordered;   // starts after everything before it
    bool announces; // its kernel says when it starts
    unsigned long long seq;
};

int batch_entry(gllmq_ctx *ctx, Scratch &S, const gllmq_matmul_desc &d, void *stream)
{
    constexpr uint32_t kElemBits = GLLMQ_DESC_ELEM_F16 | GLLMQ_DESC_ELEM_BF16;
    if (d.flags & kElemBits)
        return matmul_elem_on_scratch(ctx, S, d.w_dev, d.w_bytes, d.x_dev, d.y_dev, d.ggml_dtype, d.m, d.n, d.k,
                                      (d.flags & GLLMQ_DESC_ELEM_F16) ? GLLMQ_ELEM_F16 : GLLMQ_ELEM_BF16, stream);
    return matmul_on_scratch(ctx, S, d.w_dev, d.w_bytes, d.x_dev, d.y_dev, d.ggml_dtype, d.m, d.n, d.k, GLLMQ_ACT_F32_SPLIT, stream);
}

// The launches a batch will make, and which of them get their weights prefetched: an ordered
// launch whose kernel and whose predecessor's kernel both say when they start (the predecessor's
// start is the prefetch's cue, its own start tells a late prefetch to give up).  Nothing is
// enqueued here: single entries go through the dispatch in counting mode.
void plan_prefetch(gllmq_ctx *ctx, Scratch &S, const gllmq_matmul_desc *descs, size_t count, void *stream,
                   std::vector<BatchUnit> &units, std::vector<gq::TouchEntry> &touch)
{
    constexpr uint32_t kKnown = GLLMQ_DESC_AFTER_PREVIOUS | GLLMQ_DESC_ELEM_F16 | GLLMQ_DESC_ELEM_BF16;
    for (size_t i = 0; i < count;) {
        BatchUnit u{ i, 1, true, false, 0 };
        const size_t chain = chain_length(ctx, descs + i, count - i);
        if (chain >= 2) {
            u.len = chain;
            u.announces = true;
        } else if (!(descs[i].flags & ~kKnown)) {
            u.ordered = (descs[i].flags & GLLMQ_DESC_AFTER_PREVIOUS) != 0 || i == 0 || !ctx->batch_overlap;
            const DispatchChoice c = dispatch_choice(ctx, [&] { return batch_entry(ctx, S, descs[i], stream); });
            u.announces = c.fn != nullptr && ctx->announces.count(c.fn) != 0;
        }
        u.seq = ++ctx->launch_seq;
        units.push_back(u);
        i += u.len;
    }
    for (size_t j = 1; j < units.size(); ++j) {
        const BatchUnit &u = units[j];
        const gllmq_matmul_desc &d = descs[u.first]; // (of a chain: its first matrix; the chain's own stream carries on from there)
        if (!u.ordered || !u.announces || !units[j - 1].announces || !d.w_dev) continue;
        const size_t bytes = std::min(d.w_bytes, d.n * gllmq_row_bytes(d.ggml_dtype, d.k));
        if (bytes < (static_cast<size_t>(ctx->prefetch_min_kib) << 10)) continue;
        touch.push_back(gq::TouchEntry{ static_cast<const uint8_t *>(d.w_dev), bytes, u.seq });
    }
}

int launch_prefetch(gllmq_ctx *ctx, const std::vector<gq::TouchEntry> &touch)
{
    const uint32_t wgs = ctx->prefetch_wgs ? ctx->prefetch_wgs : static_cast<uint32_t>(ctx->num_cus);
    for (size_t at = 0; at < touch.size(); at += gq::TOUCH_MAX_ENTRIES) {
        gq::TouchParams T{};
        T.progress = ctx->progress;
        T.sink = nullptr;
        T.count = static_cast<uint32_t>(std::min<size_t>(gq::TOUCH_MAX_ENTRIES, touch.size() - at));
        T.timeout_ticks = ctx->prefetch_timeout_us * 100u; // wall_clock64() counts at 100 MHz
        T.flags = ctx->prefetch_flags;
        for (uint32_t i = 0; i < T.count; ++i) T.e[i] = touch[at + i];
        size_t size = sizeof T;
        void *config[] = { HIP_LAUNCH_PARAM_BUFFER_POINTER, &T, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END };
        GLLMQ_HIP(ctx, hipModuleLaunchKernel(ctx->touch, wgs, 1, 1, ctx->prefetch_threads, 1, 1, 0, ctx->side_stream, nullptr, config));
    }
    return GLLMQ_OK;
}

} // namespace

int gllmq_quantized_matmul_batch(gllmq_ctx *ctx, const gllmq_matmul_desc *descs, size_t count, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (count && !descs) return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_batch: NULL descriptor list");
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    // (a stream that is being captured gets ordinary launches throughout: what a capture makes of a
    // launch without order is not something to rely on; the graph's replays then run the batch's
    // kernels one after the other)
    const bool capturing = stream_is_capturing(stream);
    const bool overlap_on = ctx->batch_overlap && !capturing;
    ctx->overlap = gllmq_ctx::Overlap{};
    ctx->overlap.on = overlap_on;
    if (*ctx->chain_error) { // a chain launched earlier gave up waiting for a counter: its results are not to be trusted
        *ctx->chain_error = 0u;
        return fail(ctx, GLLMQ_ERR_HIP, "quantized_matmul_batch: an earlier chained launch timed out waiting for the entry before "
                                        "(option chain_spin_limit; is the device shared?): its outputs are invalid");
    }
    // The prefetch launch goes first, on the context's own stream (never into a capture: it is not
    // part of the caller's stream).
    std::vector<BatchUnit> units;
    std::vector<gq::TouchEntry> touch;
    if (ctx->prefetch && count >= 2 && !capturing) plan_prefetch(ctx, *S, descs, count, stream, units, touch);
    if (!touch.empty()) {
        rc = launch_prefetch(ctx, touch);
        if (rc != GLLMQ_OK) return rc;
    }
    size_t unit = 0;
    for (size_t i = 0; i < count && rc == GLLMQ_OK; ++i) {
        const gllmq_matmul_desc &d = descs[i];
        while (unit < units.size() && units[unit].first < i) ++unit;
        const bool planned = !touch.empty() && unit < units.size() && units[unit].first == i && units[unit].announces;
        ctx->call_seq = planned ? units[unit].seq : 0ull;
        // consecutive one-row matmuls of one kind run as one launch whose weight stream never stops
        const size_t chain = chain_length(ctx, descs + i, count - i);
        if (chain >= 2) {
            const int crc = run_chain(ctx, *S, descs + i, chain, stream);
            if (crc >= 0) {
                rc = crc;
                ctx->overlap = gllmq_ctx::Overlap{};
                ctx->overlap.on = overlap_on;
                i += chain - 1;
                continue;
            }
        }
        constexpr uint32_t kElemBits = GLLMQ_DESC_ELEM_F16 | GLLMQ_DESC_ELEM_BF16;
        if ((d.flags & ~(static_cast<uint32_t>(GLLMQ_DESC_AFTER_PREVIOUS) | kElemBits)) || (d.flags & kElemBits) == kElemBits) {
            rc = fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul_batch: unknown flag bits 0x%x in entry %zu", d.flags, i);
            break;
        }
        // an entry that depends on the ones before it starts a new group: its first launch is an
        // ordinary one
        ctx->overlap.entry_first = !(d.flags & GLLMQ_DESC_AFTER_PREVIOUS);
        rc = batch_entry(ctx, *S, d, stream);
    }
    ctx->call_seq = 0;
    ctx->overlap = gllmq_ctx::Overlap{};
    if (!touch.empty()) {
        // The caller's stream ends behind the prefetch: whoever waits for the stream may free the
        // weights, which the prefetch must then be through with.
        hipError_t e = hipEventRecord(ctx->side_event, ctx->side_stream);
        if (e == hipSuccess) e = hipStreamWaitEvent(static_cast<hipStream_t>(stream), ctx->side_event, 0);
        if (e != hipSuccess && rc == GLLMQ_OK) rc = fail(ctx, GLLMQ_ERR_HIP, "prefetch: %s", hipGetErrorString(e));
    }
    return rc;
}

int gllmq_chain_status(gllmq_ctx *ctx)
{
    if (!ctx || !ctx->chain_error) return 0;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const uint32_t raised = *static_cast<volatile uint32_t *>(ctx->chain_error);
    *ctx->chain_error = 0u;
    return raised ? 1 : 0;
}

int gllmq_moe_route(gllmq_ctx *ctx, const float *logits, size_t tokens, size_t experts, size_t top_k,
                    float capacity_factor, uint32_t *route_expert, float *route_weight, uint32_t *route_len,
                    uint32_t *route_pos, uint32_t *expert_counts, uint32_t *overflow, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (tokens == 0) return GLLMQ_OK;
    if (!logits || !route_expert || !route_weight || !route_len)
        return fail(ctx, GLLMQ_ERR_INVALID, "moe_route: NULL device pointer");
    if (experts == 0 || top_k == 0) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "moe_route: experts and top_k must be positive");
    if (experts > gq::ROUTE_MAX_EXPERTS || top_k > gq::ROUTE_MAX_TOP_K || tokens > 0x7FFFFFFFu / top_k)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED, "moe_route: experts = %zu (max %u), top_k = %zu (max %u) or tokens = %zu is beyond this build",
                    experts, gq::ROUTE_MAX_EXPERTS, top_k, gq::ROUTE_MAX_TOP_K, tokens);
    if (!aligned(logits, 4) || !aligned(route_expert, 4) || !aligned(route_weight, 4) || !aligned(route_len, 4))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "moe_route: buffers must be 4-byte aligned");
    gq::MoeRouteParams P{};
    P.logits = logits;
    P.route_expert = route_expert;
    P.route_weight = route_weight;
    P.route_len = route_len;
    P.route_pos = route_pos;
    P.expert_counts = expert_counts;
    P.overflow = overflow;
    P.tokens = static_cast<uint32_t>(tokens);
    P.experts = static_cast<uint32_t>(experts);
    P.top_k = static_cast<uint32_t>(top_k);
    // ExpertRouteConfig::expert_capacity (src/moe/routing.rs:53-61): the same f32 arithmetic
    float cap = std::ceil(capacity_factor * static_cast<float>(tokens) / static_cast<float>(experts));
    if (!(cap >= 0.0f)) cap = 0.0f; // negative or NaN
    if (cap > 1.0e9f) cap = 1.0e9f;
    P.capacity = static_cast<uint32_t>(cap);
    const uint32_t lds = static_cast<uint32_t>((gq::ROUTE_WAVES + 1) * experts * 4);
    if (tokens <= gq::ROUTE_FUSED_MAX_TOKENS) {
        P.phases = 3u;
        return launch(ctx, ctx->moe_route, 1, gq::ROUTE_THREADS, lds, stream, &P, sizeof P);
    }
    P.phases = 1u;
    const uint32_t grid = static_cast<uint32_t>(std::min<size_t>((tokens + gq::ROUTE_WAVES - 1) / gq::ROUTE_WAVES,
                                                                 static_cast<size_t>(ctx->num_cus) * 4));
    int rc = launch(ctx, ctx->moe_route, grid, gq::ROUTE_THREADS, lds, stream, &P, sizeof P);
    if (rc != GLLMQ_OK) return rc;
    P.phases = 2u;
    return launch(ctx, ctx->moe_route, 1, gq::ROUTE_THREADS, lds, stream, &P, sizeof P);
}

namespace {

// Carve-up of the MoE workspace (256-byte aligned pieces).
struct MoeWorkspace {
    size_t src, pos, jobs, jobs8, cnt, gu, h, o, total;
};

MoeWorkspace moe_workspace(size_t pairs, size_t hidden, size_t ffn)
{
    auto up256 = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    MoeWorkspace W{};
    size_t off = 0;
    W.src = off; off = up256(off + pairs * 4);
    W.pos = off; off = up256(off + pairs * 4);
    W.jobs = off; off = up256(off + pairs * sizeof(MoeJob));
    W.jobs8 = off; off = up256(off + pairs * sizeof(MoeJob8));
    W.cnt = off; off = up256(off + 4 * 4);
    W.gu = off; off = up256(off + pairs * 2 * ffn * 4);
    W.h = off; off = up256(off + pairs * ffn * 4);
    W.o = off; off = up256(off + pairs * hidden * 4);
    W.total = off;
    return W;
}

} // namespace

int gllmq_moe_matvec(gllmq_ctx *ctx, const void *gate, size_t gate_bytes, size_t gate_expert_stride, const void *up,
                     size_t up_bytes, size_t up_expert_stride, uint32_t dtype_gu, const void *down, size_t down_bytes,
                     size_t down_expert_stride, uint32_t dtype_dn, const float *x, float *out, size_t tokens,
                     size_t hidden, size_t ffn, size_t experts, size_t top_k, const uint32_t *route_expert,
                     const float *route_weight, const uint32_t *route_len, int relu_gate, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *fg = find_format(dtype_gu), *fd = find_format(dtype_dn);
    if (!fg || !fd)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "moe_matvec: ggml dtype %u / %u is not covered (supported: Q8_0=8, Q4_K=12, Q5_K=13, Q6_K=14)",
                    dtype_gu, dtype_dn);
    if (tokens == 0 || hidden == 0) return GLLMQ_OK;
    if (!gate || !up || !down || !x || !out || !route_expert || !route_weight || !route_len)
        return fail(ctx, GLLMQ_ERR_INVALID, "moe_matvec: NULL device pointer");
    if (ffn == 0 || experts == 0 || top_k == 0)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "moe_matvec: ffn, experts and top_k must be positive");
    const size_t pairs = tokens * top_k;
    // The plan kernel keeps the pair list and three words per expert in LDS, and a launch
    // covers at most 16384 elements of K.
    if (pairs > 16384 || experts > 4096)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED,
                    "moe_matvec: tokens*top_k = %zu (max 16384) or experts = %zu (max 4096) is beyond this build", pairs,
                    experts);
    if (hidden > 16384 || ffn > 16384)
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED, "moe_matvec: hidden = %zu / ffn = %zu beyond 16384 is not built",
                    hidden, ffn);
    if (hidden % 4 != 0 || ffn % 4 != 0)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "moe_matvec: hidden and ffn must be multiples of 4");
    const size_t rb_gu = gllmq_row_bytes(dtype_gu, hidden), rb_dn = gllmq_row_bytes(dtype_dn, ffn);
    // every expert's matrix must lie inside its buffer
    const size_t gu_each = ffn * rb_gu, dn_each = hidden * rb_dn;
    auto inside = [&](size_t bytes, size_t stride, size_t each) {
        return stride >= each && bytes >= each && (experts - 1) <= (bytes - each) / stride;
    };
    if (!inside(gate_bytes, gate_expert_stride, gu_each) || !inside(up_bytes, up_expert_stride, gu_each) ||
        !inside(down_bytes, down_expert_stride, dn_each))
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE,
                    "moe_matvec: %zu experts of %zu (gate, up) / %zu (down) bytes at strides %zu / %zu / %zu do not fit buffers of "
                    "%zu / %zu / %zu bytes", experts, gu_each, dn_each, gate_expert_stride, up_expert_stride, down_expert_stride,
                    gate_bytes, up_bytes, down_bytes);
    if (!aligned(gate, fg->w_align) || !aligned(up, fg->w_align) || rb_gu % fg->w_align != 0 ||
        gate_expert_stride % fg->w_align != 0 || up_expert_stride % fg->w_align != 0 || !aligned(down, fd->w_align) ||
        rb_dn % fd->w_align != 0 || down_expert_stride % fd->w_align != 0)
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "moe_matvec: expert weights or strides miss the alignment of their format");
    if (!aligned(x, 16) || !aligned(out, 4))
        return fail(ctx, GLLMQ_ERR_BAD_ALIGNMENT, "moe_matvec: x must be 16-byte and out 4-byte aligned");

    const MoeWorkspace W = moe_workspace(pairs, hidden, ffn);
    Scratch *Sp = nullptr;
    int rc = acquire_scratch(ctx, stream, &Sp);
    if (rc != GLLMQ_OK) return rc;
    rc = grow_scratch(ctx, *Sp, &Sp->moe, &Sp->moe_bytes, W.total, stream, "moe_matvec");
    if (rc != GLLMQ_OK) return rc;
    uint8_t *ws = static_cast<uint8_t *>(Sp->moe);
    uint32_t *pair_src = reinterpret_cast<uint32_t *>(ws + W.src);
    uint32_t *pair_pos = reinterpret_cast<uint32_t *>(ws + W.pos);
    MoeJob *jobs = reinterpret_cast<MoeJob *>(ws + W.jobs);
    MoeJob8 *jobs8 = reinterpret_cast<MoeJob8 *>(ws + W.jobs8);
    uint32_t *counters = reinterpret_cast<uint32_t *>(ws + W.cnt);
    float *gu = reinterpret_cast<float *>(ws + W.gu);
    float *h = reinterpret_cast<float *>(ws + W.h);
    float *o = reinterpret_cast<float *>(ws + W.o);

    // The streamed grouped kernels take up to four tokens per job (their ring shares the LDS with the
    // tokens' digit planes), the others up to eight.  An expert with more tokens is read once per
    // job, so the streamed form is for calls whose experts see few tokens each (at most two on
    // average: decode batches); with more, jobs of eight read the weights half as often.
    const bool streamed_jobs = ctx->use_mm8s && (ctx->moe_streamed == 2 || (ctx->moe_streamed == 1 && pairs <= 2 * experts));
    const uint32_t job_shift = streamed_jobs ? 2u : 3u;
    const uint32_t fast = pairs <= 4096 ? 1u : 0u; // per-pair placement: quadratic in the pairs, but without serial LDS walks
    {
        MoePlanParams P{ route_expert, route_len, pair_src, pair_pos, jobs, jobs8, counters, static_cast<uint32_t>(tokens),
                         static_cast<uint32_t>(top_k), static_cast<uint32_t>(experts), static_cast<uint32_t>(pairs), fast, job_shift };
        const uint32_t lds = static_cast<uint32_t>((pairs + 4 * experts + 4 + (fast ? 2 * pairs : 0)) * 4);
        rc = launch(ctx, ctx->moe_plan, 1, 256, lds, stream, &P, sizeof P);
        if (rc != GLLMQ_OK) return rc;
    }
    // Waves per job: the device takes about 8 waves per CU of these kernels; the jobs that
    // exist (at most `pairs`, typically one per routed expert) share them.
    const uint32_t job_waves = std::max<uint32_t>(16u, 4u * ctx->gemv_waves / static_cast<uint32_t>(pairs));
    // n rows of k elements per expert, experts `stride` bytes apart; the results of a pair go to
    // yout + its sorted position * y_stride.
    auto grouped = [&](const Format &f, const void *w, size_t stride, size_t rb, uint32_t n, uint32_t k, const float *xin,
                       bool x_by_token, float *yout, uint32_t y_stride) -> int {
        GemvPlan L = plan_gemv(ctx, 2, n, k, rb, job_waves);
        MoeGemvParams Q{};
        Q.g = L.P;
        Q.g.w = static_cast<const uint8_t *>(w);
        Q.g.x = xin;
        Q.g.y = yout;
        Q.g.x_vec = 1;
        Q.g.accumulate = 0;
        Q.jobs = jobs;
        Q.counters = counters;
        Q.expert_stride = stride;
        Q.wgs_per_job = L.grid;
        Q.x_by_token = x_by_token ? 1u : 0u;
        Q.x_stride = k;
        Q.y_stride = y_stride;
        const uint64_t grid = static_cast<uint64_t>(L.grid) * pairs;
        if (grid > 0x7FFFFFFFull) return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "moe_matvec: launch grid too large");
        return launch(ctx, ctx->moe_gemv[format_index(f.dtype)], static_cast<uint32_t>(grid), L.threads, L.lds, stream,
                      &Q, sizeof Q);
    };
    // Q4_K, Q5_K and Q6_K with rows of at most 16 blocks go to the int8 matrix cores, every token
    // of an expert (up to eight per job) in one pass over its weights.  `by_token`: the activation
    // rows are x[token] (gate/up), else rows by sorted position (down).
    // `up_w` != null: the gated form, n gate rows per expert at `wbase` and n up rows at `up_w`,
    // and yout receives act(gate . x) * (up . x)
    auto grouped_mm8 = [&](const Format &f, const void *wbase, size_t stride, size_t rb, uint32_t n, uint32_t k,
                           const float *xin, bool by_token, float *yout, uint32_t y_stride, const void *up_w = nullptr,
                           size_t up_stride = 0) -> int {
        const bool glu = up_w != nullptr;
        const int kind = mm8_kind(f.dtype);
        const bool q6k = kind == MM8_Q6K;
        const uint32_t groups = (k + 255u) / 256u;
        MoeMm8Params Q{};
        Q.g.w = static_cast<const uint8_t *>(wbase);
        Q.g.x = xin;
        Q.g.y = yout;
        Q.g.n = n;
        Q.g.k = k;
        Q.g.groups = groups;
        Q.g.row_bytes = static_cast<uint32_t>(rb);
        Q.g.ldx = k;
        Q.g.tiles = (n + 31u) / 32u;
        Q.jobs = jobs8;
        Q.counters = counters;
        Q.expert_stride = stride;
        Q.up = static_cast<const uint8_t *>(up_w);
        Q.up_stride = up_stride;
        Q.y_stride = y_stride;
        Q.g.glu_relu = relu_gate ? 1u : 0u;
        Q.rows = by_token ? nullptr : ctx->identity_rows;
        // upper bound of the jobs: one per expert hit, plus one per eight (four) further pairs
        const uint64_t max_jobs = std::min<uint64_t>(pairs, experts + (pairs >> job_shift));
        uint32_t slices = std::max<uint32_t>(1u, (3u * static_cast<uint32_t>(ctx->num_cus)) / (2u * static_cast<uint32_t>(std::min<uint64_t>(pairs, experts))));
        if (ctx->moe_slices) slices = ctx->moe_slices;
        const uint32_t ppt = (groups + 7u) / 8u;
        hipFunction_t fn = glu ? ctx->moe_mm8_glu_fn[kind][ppt - 1] : ctx->moe_mm8_fn[kind][ppt - 1];
        uint32_t units = Q.g.tiles; // what the slices of a job share: tiles, or groups of eight tiles
        if (q6k && groups <= 8 && ctx->moe_mm8_rows) {
            fn = ctx->moe_mm8_q6k_rows;
            units = (Q.g.tiles + 7u) / 8u;
        }
        // The streamed form (loader waves and arithmetic waves, a workgroup per CU): the kernel cuts the
        // tiles of all jobs into one run per workgroup and works the ring out per job; it must exist for
        // two and for four rows over a run of any length.
        if (streamed_jobs && ctx->moe_mm8s_fn[kind][glu ? 1 : 0] && aligned(xin, 16) && max_jobs * Q.g.tiles < 0x7FFFFFFFull) {
            const uint32_t sfmt = kind == MM8_Q6K ? 2u : kind == MM8_Q5K ? 1u : 0u;
            const uint32_t pieces = sfmt == 2 ? gq::Mm8sFormat<2>::PIECES : sfmt == 1 ? gq::Mm8sFormat<1>::PIECES : gq::Mm8sFormat<0>::PIECES;
            const uint32_t subs = sfmt == 2 ? 16u : 8u, item_bytes = 32u * pieces * 16u, lds_bytes = 160u * 1024u;
            const uint32_t items = (glu ? 2u : 1u) * Q.g.tiles * groups; // the longest piece: all tiles of a job
            gq::Mm8sLds L2, L4;
            uint32_t slots, depth;
            if (gq::mm8s_ring(groups, 2, item_bytes, items, subs, glu, lds_bytes, ctx->moe_depth, L2, slots, depth) &&
                gq::mm8s_ring(groups, 4, item_bytes, items, subs, glu, lds_bytes, ctx->moe_depth, L4, slots, depth)) {
                Q.slices = 1;
                Q.g.tile_rows = 32;
                Q.g.lds_ring = lds_bytes; // the kernel carves it up per job
                Q.g.depth = ctx->moe_depth;
                const uint64_t wgs = std::min<uint64_t>(static_cast<uint64_t>(ctx->num_cus), max_jobs * Q.g.tiles);
                return launch(ctx, ctx->moe_mm8s_fn[kind][glu ? 1 : 0], static_cast<uint32_t>(wgs),
                              (gq::MM8S_CWAVES + gq::MM8S_LOADERS) * 64, lds_bytes, stream, &Q, sizeof Q);
            }
        }
        slices = std::min(slices, units);
        Q.slices = slices;
        return launch(ctx, fn, static_cast<uint32_t>(max_jobs * slices), 512, mm8_lds_bytes(groups, 8, 4, kind), stream,
                      &Q, sizeof Q);
    };
    auto fits_mm8 = [&](const Format &f, size_t k, bool glu = false) {
        const uint32_t groups = static_cast<uint32_t>((k + 255) / 256);
        const int kind = mm8_kind(f.dtype);
        if (glu && !(ctx->moe_glu && (kind == MM8_Q4K || kind == MM8_Q5K))) return false;
        if (!(fast && ctx->use_mm8 && ctx->moe_mm8) || kind < 0 || kind >= MM8_MOE_KINDS || groups > 16 || k % 8 != 0) return false;
        if (kind == MM8_Q6K && !ctx->moe_mm8_q6k) return false;
        return mm8_lds_bytes(groups, 8, 4, kind) <= 160u * 1024u;
    };
    const uint32_t F = static_cast<uint32_t>(ffn), H = static_cast<uint32_t>(hidden);
    const bool gated = fits_mm8(*fg, hidden, true); // gate, up and the activation in one launch
    if (gated) {
        rc = grouped_mm8(*fg, gate, gate_expert_stride, rb_gu, F, H, x, true, h, F, up, up_expert_stride);
    } else {
        // an expert's up rows right behind its gate rows, both under one stride: one matrix of
        // 2 * ffn rows; otherwise the two halves of gu[pair][2 ffn] come from a launch each
        const bool stacked = static_cast<const uint8_t *>(up) == static_cast<const uint8_t *>(gate) + gu_each &&
                             up_expert_stride == gate_expert_stride;
        const bool mm8 = fits_mm8(*fg, hidden);
        for (int half = 0; half < (stacked ? 1 : 2) && rc == GLLMQ_OK; ++half) {
            const void *wb = half ? up : gate;
            const size_t st = half ? up_expert_stride : gate_expert_stride;
            const uint32_t rows = stacked ? 2u * F : F;
            if (mm8) rc = grouped_mm8(*fg, wb, st, rb_gu, rows, H, x, true, gu + half * ffn, 2u * F);
            else rc = grouped(*fg, wb, st, rb_gu, rows, H, x, true, gu + half * ffn, 2u * F);
        }
    }
    if (rc != GLLMQ_OK) return rc;
    if (!gated) {
        MoeActParams P{ gu, h, counters, F, relu_gate ? 1u : 0u };
        rc = launch2d(ctx, ctx->moe_act, (F + 255u) / 256u, static_cast<uint32_t>(pairs), 256, 0, stream, &P, sizeof P);
        if (rc != GLLMQ_OK) return rc;
    }
    if (fits_mm8(*fd, ffn)) rc = grouped_mm8(*fd, down, down_expert_stride, rb_dn, H, F, h, false, o, H);
    else rc = grouped(*fd, down, down_expert_stride, rb_dn, H, F, h, false, o, H);
    if (rc != GLLMQ_OK) return rc;
    MoeCombineParams C{ o, route_weight, route_len, pair_pos, out, static_cast<uint32_t>(tokens),
                        static_cast<uint32_t>(top_k), H };
    return launch2d(ctx, ctx->moe_combine, (H + 255u) / 256u, static_cast<uint32_t>(tokens), 256, 0, stream, &C, sizeof C);
}

int gq_quantized_matmul_on_block(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x, float *y, uint32_t dtype,
                                 size_t m, size_t n, size_t k, void *block, size_t block_bytes, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (!block || block_bytes < kScratchFixedBytes || !aligned(block, 256))
        return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul: scratch block missing, misaligned or under %zu bytes", kScratchFixedBytes);
    static_assert(kScratchArriveBytes == GQ_BLOCK_ZEROED_BYTES, "the arrival counters are the zeroed head of the block");
    Scratch S;
    S.stream = static_cast<hipStream_t>(stream);
    S.fixed = true;
    carve_fixed(S, block);
    S.mmf = static_cast<uint8_t *>(block) + kScratchFixedBytes;
    S.mmf_bytes = block_bytes - kScratchFixedBytes;
    return matmul_on_scratch(ctx, S, w, w_bytes, x, y, dtype, m, n, k, GLLMQ_ACT_F32_SPLIT, stream);
}

namespace {

// Device copy of a host weight slice, uploaded on first sight and kept (call_mutex held).  The key is
// the slice itself (address and length): the reference treats weights as immutable once loaded
// and keeps its uploaded blob by length alone (src/compat/hip_backend.rs:141-156).
int cached_weights(gllmq_ctx *ctx, const void *host, size_t bytes, void **dev)
{
    ++ctx->use_counter;
    for (CachedWeights &W : ctx->weights)
        if (W.host == host && W.bytes == bytes) {
            W.last_use = ctx->use_counter;
            *dev = W.dev;
            return GLLMQ_OK;
        }
    GLLMQ_HIP(ctx, hipSetDevice(ctx->device));
    // make room: least recently used first
    size_t held = 0;
    for (const CachedWeights &W : ctx->weights) held += W.bytes;
    while (!ctx->weights.empty() && held + bytes > ctx->weights_cache_limit) {
        size_t lru = 0;
        for (size_t i = 1; i < ctx->weights.size(); ++i)
            if (ctx->weights[i].last_use < ctx->weights[lru].last_use) lru = i;
        GLLMQ_HIP(ctx, hipDeviceSynchronize());
        (void)hipFree(ctx->weights[lru].dev);
        held -= ctx->weights[lru].bytes;
        ctx->weights.erase(ctx->weights.begin() + static_cast<long>(lru));
    }
    CachedWeights W;
    W.host = host;
    W.bytes = bytes;
    W.last_use = ctx->use_counter;
    GLLMQ_HIP(ctx, hipMalloc(&W.dev, bytes));
    hipError_t e = hipMemcpy(W.dev, host, bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(W.dev);
        return fail(ctx, GLLMQ_ERR_HIP, "weight upload: %s", hipGetErrorString(e));
    }
    ++ctx->weight_uploads;
    ctx->weights.push_back(W);
    *dev = W.dev;
    return GLLMQ_OK;
}

} // namespace

void gllmq_weights_forget(gllmq_ctx *ctx, const void *host)
{
    if (!ctx) return;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    for (size_t i = 0; i < ctx->weights.size();) {
        if (host == nullptr || ctx->weights[i].host == host) {
            (void)hipDeviceSynchronize();
            (void)hipFree(ctx->weights[i].dev);
            ctx->weights.erase(ctx->weights.begin() + static_cast<long>(i));
        } else {
            ++i;
        }
    }
}

uint64_t gllmq_weight_uploads(const gllmq_ctx *ctx) { return ctx ? ctx->weight_uploads : 0; }

int gllmq_reserve_matmul(gllmq_ctx *ctx, uint32_t dtype, size_t m, size_t n, size_t k, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    if (!find_format(dtype))
        return fail(ctx, GLLMQ_ERR_UNIMPLEMENTED, "reserve_matmul: ggml dtype %u is not covered", dtype);
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK || m == 0 || n == 0 || k == 0) return rc;
    // the GEMM is the only matmul kernel family whose scratch depends on the shape; it may take
    // any call of 3 rows and more
    if (m < 3) return GLLMQ_OK;
    // (either form of it: which one runs also depends on the activation pointer's alignment)
    size_t need = plan_mmf(ctx, m, n, k).need;
    const MmfsPlan Ls = plan_mmfs(ctx, *find_format(dtype), m, n, k);
    if (Ls.ok) need = std::max(need, Ls.need);
    return grow_scratch(ctx, *S, &S->mmf, &S->mmf_bytes, need, stream, "reserve_matmul");
}

int gllmq_reserve_ffn(gllmq_ctx *ctx, uint32_t dtype_gate_up, uint32_t dtype_down, size_t m, size_t hidden, size_t ffn,
                      void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    int rc = gllmq_reserve_matmul(ctx, dtype_gate_up, m, 2 * ffn, hidden, stream);
    if (rc == GLLMQ_OK) rc = gllmq_reserve_matmul(ctx, dtype_down, m, hidden, ffn, stream);
    if (rc != GLLMQ_OK || m == 0 || hidden == 0 || ffn == 0) return rc;
    Scratch *S = nullptr;
    rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK) return rc;
    return grow_scratch(ctx, *S, &S->ffn, &S->ffn_bytes, ffn_scratch_bytes(m, ffn), stream, "reserve_ffn");
}

int gllmq_reserve_moe(gllmq_ctx *ctx, size_t tokens, size_t top_k, size_t hidden, size_t ffn, void *stream)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    Scratch *S = nullptr;
    int rc = acquire_scratch(ctx, stream, &S);
    if (rc != GLLMQ_OK || tokens == 0 || top_k == 0) return rc;
    return grow_scratch(ctx, *S, &S->moe, &S->moe_bytes, moe_workspace(tokens * top_k, hidden, ffn).total, stream,
                        "reserve_moe");
}

int gllmq_dequantize_host(gllmq_ctx *ctx, const void *blocks, size_t n_bytes, float *out, size_t n_out,
                          uint32_t dtype)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *f = find_format(dtype);
    if (!f) return gllmq_dequantize(ctx, blocks, n_bytes, out, n_out, dtype, nullptr);
    const size_t nb = std::min(n_bytes / f->block_bytes, n_out / f->block_size);
    if (nb == 0) return GLLMQ_OK;
    void *d_in = nullptr, *d_out = nullptr;
    int rc = cached_weights(ctx, blocks, nb * f->block_bytes, &d_in);
    if (rc != GLLMQ_OK) return rc;
    hipError_t e = hipMalloc(&d_out, nb * f->block_size * sizeof(float));
    if (e != hipSuccess) rc = fail(ctx, GLLMQ_ERR_HIP, "hipMalloc: %s", hipGetErrorString(e));
    if (rc == GLLMQ_OK)
        rc = gllmq_dequantize(ctx, d_in, nb * f->block_bytes, static_cast<float *>(d_out), nb * f->block_size,
                              dtype, nullptr);
    if (rc == GLLMQ_OK &&
        (e = hipMemcpy(out, d_out, nb * f->block_size * sizeof(float), hipMemcpyDeviceToHost)) != hipSuccess)
        rc = fail(ctx, GLLMQ_ERR_HIP, "hipMemcpy D2H: %s", hipGetErrorString(e));
    (void)hipFree(d_out);
    return rc;
}

int gllmq_quant_gather_host(gllmq_ctx *ctx, const void *table, size_t table_bytes, uint32_t dtype, size_t vocab,
                            size_t hidden, const uint32_t *ids, size_t count, float scale, float *out)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *f = find_format(dtype);
    if (!f || count == 0 || hidden == 0 || !table || !ids || !out || hidden % 4 != 0 ||
        table_bytes < vocab * gllmq_row_bytes(dtype, hidden)) // the device entry point reports these
        return gllmq_quant_gather(ctx, table, table_bytes, dtype, vocab, hidden, ids, count, scale, out, nullptr);
    for (size_t i = 0; i < count; ++i)
        if (ids[i] >= vocab)
            return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quant_gather: id %u at position %zu is outside the %zu-row table",
                        ids[i], i, vocab);
    const size_t tb = vocab * gllmq_row_bytes(dtype, hidden);
    void *d_t = nullptr, *d_i = nullptr, *d_o = nullptr;
    int rc = cached_weights(ctx, table, tb, &d_t);
    if (rc != GLLMQ_OK) return rc;
    hipError_t e = hipMalloc(&d_i, count * sizeof(uint32_t));
    if (e == hipSuccess) e = hipMalloc(&d_o, count * hidden * sizeof(float));
    if (e == hipSuccess) e = hipMemcpy(d_i, ids, count * sizeof(uint32_t), hipMemcpyHostToDevice);
    rc = e == hipSuccess ? GLLMQ_OK : fail(ctx, GLLMQ_ERR_HIP, "quant_gather: %s", hipGetErrorString(e));
    if (rc == GLLMQ_OK)
        rc = gllmq_quant_gather(ctx, d_t, tb, dtype, vocab, hidden, static_cast<const uint32_t *>(d_i), count, scale,
                                static_cast<float *>(d_o), nullptr);
    if (rc == GLLMQ_OK && (e = hipMemcpy(out, d_o, count * hidden * sizeof(float), hipMemcpyDeviceToHost)) != hipSuccess)
        rc = fail(ctx, GLLMQ_ERR_HIP, "hipMemcpy D2H: %s", hipGetErrorString(e));
    (void)hipFree(d_i);
    (void)hipFree(d_o);
    return rc;
}

int gllmq_quantized_matmul_host(gllmq_ctx *ctx, const void *w, size_t w_bytes, const float *x, float *y,
                                uint32_t dtype, size_t m, size_t n, size_t k)
{
    if (!ctx) return GLLMQ_ERR_INVALID;
    std::lock_guard<std::recursive_mutex> call(ctx->call_mutex);
    const Format *f = find_format(dtype);
    if (!f) return gllmq_quantized_matmul(ctx, w, w_bytes, x, y, dtype, m, n, k, nullptr);
    if (m == 0 || n == 0) return GLLMQ_OK;
    if (!w || !x || !y) return fail(ctx, GLLMQ_ERR_INVALID, "quantized_matmul: NULL pointer");
    const size_t need = n * gllmq_row_bytes(dtype, k);
    if (w_bytes < need)
        return fail(ctx, GLLMQ_ERR_BAD_SHAPE, "quantized_matmul: weight buffer has %zu bytes, need %zu", w_bytes, need);
    void *d_w = nullptr, *d_x = nullptr, *d_y = nullptr;
    int rc = cached_weights(ctx, w, need, &d_w);
    if (rc != GLLMQ_OK) return rc;
    hipError_t e;
    if ((e = hipMalloc(&d_x, m * k * sizeof(float))) != hipSuccess || (e = hipMalloc(&d_y, m * n * sizeof(float))) != hipSuccess)
        rc = fail(ctx, GLLMQ_ERR_HIP, "hipMalloc: %s", hipGetErrorString(e));
    if (rc == GLLMQ_OK && (e = hipMemcpy(d_x, x, m * k * sizeof(float), hipMemcpyHostToDevice)) != hipSuccess)
        rc = fail(ctx, GLLMQ_ERR_HIP, "hipMemcpy H2D: %s", hipGetErrorString(e));
    if (rc == GLLMQ_OK)
        rc = gllmq_quantized_matmul(ctx, d_w, need, static_cast<const float *>(d_x), static_cast<float *>(d_y),
                                    dtype, m, n, k, nullptr);
    if (rc == GLLMQ_OK && (e = hipMemcpy(y, d_y, m * n * sizeof(float), hipMemcpyDeviceToHost)) != hipSuccess)
        rc = fail(ctx, GLLMQ_ERR_HIP, "hipMemcpy D2H: %s", hipGetErrorString(e));
    (void)hipFree(d_x);
    (void)hipFree(d_y);
    return rc;
}

} // extern "C"
