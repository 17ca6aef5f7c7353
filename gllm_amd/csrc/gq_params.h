// Kernel parameter blocks and LDS layouts of the library, shared by the gfx950 kernels
// (gllmq_kernels.hip) and the host launcher (gllmq_host.cpp): one definition, so the bytes the
// host hands to hipModuleLaunchKernel are the struct the kernel reads.
#ifndef GQ_PARAMS_H
#define GQ_PARAMS_H

#include <stdint.h>

#if defined(__HIP__)
#define GQ_HD __host__ __device__
#else
#define GQ_HD
#endif

namespace gq {

struct GemvParams {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t n;          // weight rows = outputs
    uint32_t k;          // elements per row (activations beyond k read as zero)
    uint32_t groups;     // 256-element groups per row = ceil(k / 256)
    uint32_t row_bytes;  // bytes between rows
    uint32_t ks;         // waves that share one row (K split)
    uint32_t rps;        // rows side by side in one wave (1 when a row fills the wave)
    uint32_t rows_per_wg;
    uint32_t ldx;        // elements between activation rows
    uint32_t ldy;        // elements between output rows
    uint32_t x_vec;      // activation rows are 16-byte aligned: vector loads allowed
    uint32_t accumulate; // add to y instead of overwriting it (K handled in several launches)
    uint32_t prep_words; // integer-dot kernels: 32-bit words of LDS holding the prepared activations
    uint32_t act_bf16;   // integer-dot kernels: round activations to bf16 before use
    uint32_t elem;       // integer-dot kernels: element type of x and y (ELEM_F32 / ELEM_F16 / ELEM_BF16)
    uint32_t glu, glu_off; // integer-dot kernels: x[i] = act(x[i]) * x[i + glu_off] (0 off, 1 SiLU, 2 SiLU behind a ReLU)
    // kernels that end in the greedy token choice: one candidate per workgroup (argmax_key); the
    // workgroup that finishes last (ticket counts them and is left at 0) picks among them
    uint64_t *keys;
    uint32_t *ticket;
    uint32_t *token; // the choice (ARGMAX_NONE: no candidate)
    float *value;    // null, or the chosen logit (NaN: none)
};

struct Mm8Params {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t n;         // weight rows
    uint32_t k;         // elements per row
    uint32_t groups;    // 256-element blocks per row
    uint32_t row_bytes; // bytes between rows
    uint32_t m;         // activation rows (<= 2 * PAIRS of the kernel)
    uint32_t ldx, ldy;
    uint32_t tiles;     // ceil(n / 32)
    uint32_t grid;      // workgroups launched (kept beside the other fields so one kernarg line holds all)
    uint32_t act_bf16;  // round activations to bf16 before use
    const uint32_t *xrows; // row of x (in units of ldx) behind each of the m activation rows: 0..m-1, or gathered rows
    // gated form only (gq_mm8_glu_*): the up rows, and whether the gate passes a ReLU ahead of the SiLU
    const uint8_t *w2;
    uint32_t glu_relu;
    // K split (plain kernels only; 0 or 1 = off): `ksplit` consecutive workgroups share a tile list,
    // workgroup s of them multiplies blocks [s * kslice_groups, (s + 1) * kslice_groups) of every
    // row and writes its sums to part[s][m][n]; the one that finishes last adds the slices up in
    // order (arrive[tile list] counts the finished ones and is left at 0).
    uint32_t ksplit, kslice_groups;
    uint32_t elem;      // element type of x and y (ELEM_F32 / ELEM_F16 / ELEM_BF16); the slice sums stay f32
    float *part;
    uint32_t *arrive;
    // streamed kernels (mm8s.hip.inc) only, all worked out by the host so that a loader wave's
    // way to its first load is short: weight rows per workgroup, rows per tile (<= 32: a
    // workgroup's rows are cut into tiles of equal height), item slots of the LDS ring (a
    // multiple of the loader waves unless the ring holds every item), tiles of a full
    // workgroup and of the last one, rows of the last one, the LDS offsets of the counters
    // and of the ring, and the items a loader keeps unconfirmed (1 .. MM8S_MAX_DEPTH)
    uint32_t rows_per_wg, tile_rows, ring_slots, wg_tiles, last_wg_tiles, last_wg_rows, lds_ctrl, lds_ring, depth;
    // activations that are the gated product of two f32 vectors (the input of a feed-forward
    // block's down projection): x[i] = act(x[i]) * x[i + glu_off]; glu = 0 off, 1 SiLU, 2 SiLU behind a ReLU
    uint32_t glu, glu_off;
    // streamed kernels: null, or the word that says which launch of the context has started (the
    // weight prefetch of the launch behind this one waits for it): workgroup 0 raises it to
    // `progress_seq` on its way in
    unsigned long long *progress;
    unsigned long long progress_seq;
};

// The weight prefetch that runs beside a sequence of dependent launches (touch.hip.inc): for each
// entry, in order, wait until launch number `seq - 1` of the context has started (`progress`, see
// Mm8Params), then pull the entry's bytes into the memory-side cache by reading one word of every
// 128-byte line.  An entry whose own launch has already started, or whose wait runs out after
// `timeout_ticks` of the 100 MHz clock, is skipped: the prefetch never holds anything up.
constexpr uint32_t TOUCH_MAX_ENTRIES = 32;
struct TouchEntry {
    const uint8_t *w;
    unsigned long long bytes;
    unsigned long long seq;
};
struct TouchParams {
    const unsigned long long *progress;
    uint32_t *sink;          // null (a place the words read would go to if they were ever needed)
    uint32_t count, timeout_ticks;
    uint32_t flags, pad;     // bit 0: wait as usual but read nothing (for measurements)
    TouchEntry e[TOUCH_MAX_ENTRIES];
};

constexpr uint32_t MM8_SPLIT_MAX_LISTS = 256;        // tile lists (workgroups per slice) of a K-split launch
constexpr uint32_t MM8_SPLIT_PART_FLOATS = 1u << 20; // slices * activation rows * n of a K-split launch (4 MiB)

constexpr int MM8_WAVES = 8;
constexpr int MM8_THREADS = 64 * MM8_WAVES;
constexpr int MM8_LOADS = 5;            // 16-byte loads per lane for one 32-row block tile (4.5 used)
constexpr int MM8_STAGE_BYTES = 5120;   // 32 rows x 144 bytes, rounded up to whole wave loads

// What differs between the two formats of mm8.hip.inc.  Q5_K is Q4_K with a fifth bit per quant
// (32 bytes of qh between the header and the nibbles): same sub-blocks, scales and mins.
template <int FMT> struct Mm8Format;
template <> struct Mm8Format<0> { // Q4_K
    static constexpr uint32_t BLOCK = 144, CHUNKS = 9, QS = 16, STAGE = MM8_STAGE_BYTES;
    static constexpr int LOADS = MM8_LOADS;
};
template <> struct Mm8Format<1> { // Q5_K
    static constexpr uint32_t BLOCK = 176, CHUNKS = 11, QS = 48, STAGE = 6144; // 32 rows x 176 bytes, rounded up
    static constexpr int LOADS = 6;                                           // 5.5 used
};

// What the streamed kernels (mm8s.hip.inc) need to know of a format: bytes of a block in memory,
// 16-byte pieces a block's row is fetched as (Q6_K blocks are 210 bytes and only 2-byte aligned:
// 13 pieces at 16 p and a fourteenth at 194, so no load runs past a block), wave-loads of a
// 32-row item, sub-block sums the preparation keeps per block.  In LDS a row of an item is its
// pieces side by side, PIECES * 16 bytes.
template <int FMT> struct Mm8sFormat;
template <> struct Mm8sFormat<0> { static constexpr uint32_t BLOCK = 144, PIECES = 9, SUBS = 8; };   // Q4_K
template <> struct Mm8sFormat<1> { static constexpr uint32_t BLOCK = 176, PIECES = 11, SUBS = 8; };  // Q5_K
template <> struct Mm8sFormat<2> { static constexpr uint32_t BLOCK = 210, PIECES = 14, SUBS = 16; }; // Q6_K
template <> struct Mm8sFormat<3> { static constexpr uint32_t BLOCK = 272, PIECES = 17, SUBS = 0; };   // Q8_0: a group of 8 blocks of 34 bytes (K a multiple of 256)
GQ_HD constexpr uint32_t mm8s_piece_offset(int fmt, uint32_t piece) { return (fmt == 2 && piece == 13u) ? 194u : 16u * piece; }

// LDS carve-up (bytes) of the int8 matrix-core kernels.
struct Mm8Lds {
    uint32_t plane_stride; // bytes between digit planes
    uint32_t planes;       // offset of [3 * m][plane_stride]
    uint32_t sums;         // offset of float [m][groups][8]: sum of X per sub-block
    uint32_t scales;       // offset of float [m][groups]: 2^e per block (NaN if poisoned)
    uint32_t red;          // offset of float [2][MM8_WAVES][PAIRS][64]
    uint32_t stage;        // offset of [MM8_WAVES][MM8_STAGE_BYTES]: one weight block tile per wave
    uint32_t total;
};

// `subs`: sub-block sums kept per 256-element block (8 of 32 elements for Q4_K, 16 of 16 for
// Q6_K, none for Q8_0); `stage_bytes`: one wave's weight stage.
GQ_HD inline Mm8Lds mm8_lds_layout(uint32_t groups, uint32_t m, uint32_t pairs, uint32_t subs = 8u,
                                   uint32_t stage_bytes = MM8_STAGE_BYTES)
{
    Mm8Lds L;
    L.plane_stride = groups * 256u + 16u; // +16 staggers the planes over the LDS banks
    L.planes = 0;
    L.sums = L.planes + 3u * m * L.plane_stride;
    L.scales = L.sums + m * groups * subs * 4u;
    L.red = (L.scales + m * groups * 4u + 15u) & ~15u;
    L.stage = L.red + 2u * MM8_WAVES * pairs * 64u * 4u;
    L.total = L.stage + MM8_WAVES * stage_bytes;
    return L;
}

// Streamed form of the int8 matrix-core kernels (mm8s.hip.inc): loader waves and arithmetic waves.
constexpr int MM8S_CWAVES = 8;      // arithmetic waves
#ifndef GQ_MM8S_LOADERS
#define GQ_MM8S_LOADERS 4
#endif
constexpr int MM8S_LOADERS = GQ_MM8S_LOADERS; // loader waves
constexpr int MM8S_RED_BUFS = 4;    // tiles whose partial sums can be waiting in LDS
// Items a loader keeps unconfirmed (its depth D, chosen per launch: what is in flight per CU,
// not the item count, is what keeps the memory system busy, and items of low tiles are small).
// A loader's outstanding wave-loads are counted by a 6-bit counter: D times the wave-loads of
// an item (at most 7) stays below 64.
constexpr uint32_t MM8S_MAX_DEPTH = 6;
constexpr uint32_t MM8S_DEPTH_BYTES = 8192; // a loader keeps about this much unconfirmed
// A consumer sees item i once its loader has requested D more items of its own, that is item
// i + D * MM8S_LOADERS, and that request waits for the slot of item i + D * MM8S_LOADERS - slots
// to be free: with slots > D * MM8S_LOADERS every wait is for an item with a smaller number and
// the chain ends.  Half as many again keep the stream going while items are being multiplied.
inline GQ_HD uint32_t mm8s_min_slots(uint32_t depth) { return depth * MM8S_LOADERS + MM8S_LOADERS * ((depth + 1u) / 2u); }

struct Mm8sCtrl {                    // counters in LDS, all start at zero
    uint32_t landed[8];              // per loader: items whose bytes are in LDS
    uint32_t done[MM8S_CWAVES];      // per arithmetic wave: items consumed
    uint32_t arrived[MM8S_RED_BUFS]; // per partial-sum buffer: waves that left their sums
    uint32_t reduced;                // tiles summed and stored
    uint32_t finished;               // K split: arithmetic waves whose slice sums have reached coherent memory
    uint32_t pad[2];
};

// LDS carve-up of the streamed kernels: the preparation's planes, sums and scales as in
// mm8_lds_layout, then the counters, the partial sums and the ring of item slots.
struct Mm8sLds {
    Mm8Lds prep;
    uint32_t ctrl, red, ring, total;
};

// The folded form of the streamed kernels (one activation row, tiles of at most 16 weight rows):
// an item is a pair of blocks of the tile, blocks 16 q + i and 16 q + 8 + i (i < 8) being pair
// 8 q + i, so that the arithmetic wave of a pair (pair mod 8) is the wave of both of its blocks
// (block mod 8), as in the form that goes block by block: the same wave prepares the activations
// of a block either way.  A row whose last group of 16 blocks has 8 or fewer ends in pairs without
// a second block.
GQ_HD inline uint32_t mm8s_fold_pairs(uint32_t groups) { return 8u * (groups / 16u) + (groups % 16u < 8u ? groups % 16u : 8u); }
GQ_HD inline uint32_t mm8s_fold_first(uint32_t pair) { return 16u * (pair >> 3) + (pair & 7u); }

// `glu`: the gated kernels keep the sums of a gate tile (pairs x 64 floats) behind the partial sums
// until the up tile of the same rows is summed.
GQ_HD inline Mm8sLds mm8s_lds_layout(uint32_t groups, uint32_t m, uint32_t pairs, uint32_t item_bytes, uint32_t slots,
                                     uint32_t subs = 8u, bool glu = false)
{
    Mm8sLds L;
    L.prep = mm8_lds_layout(groups, m, pairs, subs, 0u);
    L.ctrl = (L.prep.red + 15u) & ~15u; // the area of mm8.hip.inc's partial sums and stages is not used here
    L.red = L.ctrl + static_cast<uint32_t>(sizeof(Mm8sCtrl));
    L.ring = (L.red + MM8S_RED_BUFS * MM8S_CWAVES * pairs * 64u * 4u + (glu ? pairs * 64u * 4u : 0u) + 1023u) & ~1023u;
    L.total = L.ring + slots * item_bytes;
    return L;
}

// Ring and loader depth of a streamed launch for `m` activation rows (1..4) whose items, `items`
// per workgroup of `item_bytes` each, share `lds_bytes` of LDS with the preparation of `groups`
// blocks: one or two rows keep one item per loader unconfirmed, three and four about
// MM8S_DEPTH_BYTES.  False when the ring would be too short for the loaders to run ahead.
// `want_depth` != 0: that many items per loader instead (a long stream gains from more of them).
GQ_HD inline bool mm8s_ring(uint32_t groups, uint32_t m, uint32_t item_bytes, uint32_t items, uint32_t subs, bool glu,
                            uint32_t lds_bytes, uint32_t want_depth, Mm8sLds &L, uint32_t &slots, uint32_t &depth)
{
    const uint32_t pairs = m <= 2u ? 1u : 2u;
    L = mm8s_lds_layout(groups, m, pairs, item_bytes, 0u, subs, glu);
    if (L.total + item_bytes > lds_bytes) return false;
    slots = (lds_bytes - L.total) / item_bytes;
    if (slots >= items) slots = items;
    else slots -= slots % MM8S_LOADERS; // a reused ring is a whole number of rounds of the loaders
    depth = 1u;
    if (pairs > 1u) {
        depth = (MM8S_DEPTH_BYTES + item_bytes / 2u) / item_bytes;
        depth = depth < 2u ? 2u : (depth > MM8S_MAX_DEPTH ? MM8S_MAX_DEPTH : depth);
    }
    if (want_depth) depth = want_depth > MM8S_MAX_DEPTH ? MM8S_MAX_DEPTH : want_depth;
    while (depth > (pairs > 1u ? 2u : 1u) && slots < items && slots < mm8s_min_slots(depth)) --depth;
    return slots >= items || slots >= mm8s_min_slots(depth);
}

// Q6_K flavour (mm8_q6k.hip.inc)
constexpr int MM8Q6_LOADS = 7;             // 16-byte loads per lane for one 32-row block tile (32 x 14 pieces)
constexpr int MM8Q6_ROW_STRIDE = 240;      // bytes between rows in the stage: 224 used, padded against bank conflicts
constexpr int MM8Q6_STAGE_BYTES = 32 * MM8Q6_ROW_STRIDE;

// Q8_0 flavour (mm8_q8_0.hip.inc): 8 blocks of 34 bytes per 256 elements
constexpr int MM8Q8_LOADS = 9;             // 16-byte loads per lane for one 32-row group tile (32 x 17 pieces, 8.5 used)
constexpr int MM8Q8_ROW_STRIDE = 272;      // bytes between rows in the stage: the 8 blocks as they lie in memory
constexpr int MM8Q8_STAGE_BYTES = 32 * MM8Q8_ROW_STRIDE;

struct MmfParams {
    const uint8_t *w;
    const float *x;
    float *y;
    uint8_t *ximg;       // [groups] images of the prepared activations, MmfLds<MT>::image bytes apart
    float *partial;      // [ksplit][m][n] when ksplit > 1
    uint32_t n, k, groups, row_bytes, m, ldx, ldy;
    uint32_t row_tiles;        // ceil(n / 256)
    uint32_t ksplit;           // workgroups per row tile
    uint32_t blocks_per_split; // 256-element blocks of K per workgroup
    uint32_t act_bf16;
    uint32_t elem;             // element type of y (ELEM_F32 / ELEM_F16 / ELEM_BF16); partial sums stay f32
};

constexpr int MMF_WAVES = 8;
constexpr int MMF_ST = 1;                                  // 32-row sub-tiles per wave
constexpr int MMF_THREADS = 64 * MMF_WAVES;
constexpr int MMF_TILE_ROWS = 32 * MMF_ST * MMF_WAVES;     // weight rows per workgroup
constexpr int MMF_PREP_THREADS = 1024;                     // threads that prepare one block of K
constexpr int MMF_XROW_BYTES = 256 * 2 + 16;   // one activation row of a block in LDS (f16), padded
constexpr int MMF_STAGE_BYTES = 5120;          // one 32-row sub-tile of one block, as fetched

// FMT: 0 = Q4_K (144-byte blocks, 5 KiB per wave stage), 1 = Q5_K (176 bytes, 6 KiB), 2 = Q6_K, 3 = Q8_0.
template <int FMT> struct MmfFormat;
template <> struct MmfFormat<0> { static constexpr uint32_t BLOCK = 144, CHUNKS = 9, QS = 16, STAGE = 5120; static constexpr int LOADS = 5; };
template <> struct MmfFormat<1> { static constexpr uint32_t BLOCK = 176, CHUNKS = 11, QS = 48, STAGE = 6144; static constexpr int LOADS = 6; };
template <> struct MmfFormat<2> { static constexpr uint32_t STAGE = MM8Q6_STAGE_BYTES; }; // Q6_K (mmf_q6k.hip.inc): 7.5 KiB
template <> struct MmfFormat<3> { static constexpr uint32_t STAGE = MM8Q8_STAGE_BYTES; }; // Q8_0 (mmf_q8_0.hip.inc): 8.5 KiB

// LDS carve-up for MT 32-row activation tiles.  The first `image` bytes are the block image
// that gq_mmf_prep_* writes and the GEMM copies verbatim: hi plane, sub-block sums, inverse
// scales, lo plane, padded to whole rounds of one 16-byte chunk per thread.
template <int MT, int FMT = 0>
struct MmfLds {
    static constexpr uint32_t rows = 32u * MT;
    static constexpr uint32_t hi = 0;
    static constexpr uint32_t sums = hi + rows * MMF_XROW_BYTES; // [rows][16] f16: 8 hi, 8 lo
    static constexpr uint32_t inv = sums + rows * 32u;           // [rows] f32
    static constexpr uint32_t lo = inv + rows * 4u;
    static constexpr uint32_t round = MMF_THREADS * 16u;
    static constexpr uint32_t loads_hi = (lo + round - 1u) / round;                           // copy rounds without the lo plane
    static constexpr uint32_t loads_all = (lo + rows * MMF_XROW_BYTES + round - 1u) / round;  // with it
    static constexpr uint32_t image = loads_all * round;
    static constexpr uint32_t stages = MMF_WAVES * MMF_ST * MmfFormat<FMT>::STAGE; // one weight stage per wave
    // One image and one set of stages, or (when two of each fit the 160 KiB of a CU) two that
    // take turns: image p at p * image, stage set p behind the images.
    static constexpr bool twice = 2u * (image + stages) <= 160u * 1024u;
    static constexpr uint32_t stage = (twice ? 2u : 1u) * image; // [twice ? 2 : 1][waves][MMF_ST][MMF_STAGE_BYTES]
    static constexpr uint32_t total = stage + (twice ? 2u : 1u) * stages;
};

// A chain of streamed one- or two-row matmuls in one launch (mm8c.hip.inc).
constexpr int MM8C_CWAVES = 8;             // arithmetic waves (MM8_WAVES: the preparation is the same code)
constexpr int MM8C_LOADERS = 4;            // loader waves
constexpr int MM8C_RED_BUFS = 4;           // tiles whose partial sums can be waiting in LDS
constexpr uint32_t MM8C_MAX_SLOTS = 32;    // ring slots (a counter each)
constexpr uint32_t MM8C_MAX_ENTRIES = 32;  // matmuls per launch
struct Mm8ChainEntry {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t n, ldy;
    // the entry's geometry, worked out by the host as for the streamed kernels: weight rows per
    // workgroup, workgroups that take part, tile height, tiles of a full and of the last
    // workgroup, rows of the last workgroup; flags: bit 0 = its x is (part of) the y of the entry
    // before it, read from the mailbox, bit 1 = the entry behind it reads this one's y (so this one
    // posts its outputs there), bit 2 = its items are pairs of blocks (one activation row, tiles
    // of at most 16 rows)
    uint32_t rows_per_wg, grid, tile_rows, wg_tiles, last_wg_tiles, last_wg_rows, flags;
    // mailbox places (in pairs, see Mm8ChainParams::box): where this entry posts output row 0 (rows
    // `n` apart), and where its own activation row 0 was posted by the entry before (rows `x_ld` apart)
    uint32_t box_at, x_at, x_ld, pad;
};
struct Mm8ChainParams {
    uint32_t count, launched;     // entries, workgroups of the launch (the largest `grid`)
    uint32_t k, groups, row_bytes, m, ldx, act_bf16;
    uint32_t ring_slots, slot_bytes, depth, lds_ctrl, lds_ring, spin_limit;
    // Entries that read the output of the one before them inside the launch: every output of such
    // a producer is also posted as one 64-bit word (epoch << 32 | value bits) with a device-scope
    // store, entry e under epoch `epoch0 + e`; a reader loads the words it needs until all carry the
    // producer's epoch.  A word says by itself that its value is there, so nobody waits for stores
    // to be acknowledged, nothing is counted, and nothing is set back: epochs are the context's own
    // count of chained entries, no earlier launch used them, and every entry of a launch has places
    // of its own.  Null when no entry waits.
    unsigned long long *box;
    uint32_t epoch0, pad0;
    uint32_t *error;              // host-visible word, set to 1 when a reader's wait ran out
    unsigned long long *progress; // as in Mm8Params
    unsigned long long progress_seq;
    Mm8ChainEntry e[MM8C_MAX_ENTRIES];
};

// Streamed form of the Q4_K / Q5_K GEMM (mmfs.hip.inc): takes Mm8Params like the streamed int8
// kernels, whose loader it shares (x holds the activation images, groups all blocks of K,
// kslice_groups the blocks of a workgroup's slice of K, grid the row ranges).
// Its activation image of one block of K and 32 rows, in the order the lanes hold it: for each of
// the 16 K steps of the block the 64 lanes' 16-byte operands (lane = row + 32 * half of the step)
// one after the other, hi plane then lo plane; the sub-block sums as the operand of the min term
// (hi sums for the lanes of half 0, lo sums for half 1); the rows' inverse scales.  Every register
// of a wave is then one contiguous 1 KiB load.
struct MmfLanes {
    static constexpr uint32_t hi = 0, lo = 16u * 1024u, sums = 32u * 1024u, inv = 33u * 1024u, image = 34u * 1024u;
};
constexpr int MMFS_CWAVES = 4;  // arithmetic waves = blocks of K per workgroup
constexpr int MMFS_LOADERS = 4; // loader waves (MM8S_LOADERS: the loader is the same code)
constexpr int MMFS_RED_BUFS = 3; // tiles whose block sums can be waiting in LDS
static_assert(MMFS_LOADERS == MM8S_LOADERS, "mm8s_min_slots() is worked out for that many loaders");

// The streamed GEMM whose waves prepare their own activations (mmfr.hip.inc).
constexpr int MMFR_CWAVES = 8;   // arithmetic waves
constexpr int MMFR_LOADERS = 4;  // loader waves (MM8S_LOADERS: the loader is the same code)
constexpr int MMFR_RED_BUFS = 3; // tiles whose block sums can be waiting in LDS
constexpr uint32_t MMFR_RED_WAVE = 2u * 64u * 16u; // bytes of a tile's sums in LDS per wave: [column tile][lane] float4

struct MmfPrepParams {
    const float *x;
    uint8_t *ximg;
    uint32_t m, k, ldx, act_bf16;
    uint32_t elem; // element type of x
    uint32_t glu, glu_off; // x[i] = act(x[i]) * x[i + glu_off] (0 off, 1 SiLU, 2 SiLU behind a ReLU)
};

struct MmfReduceParams {
    const float *partial; // [ksplit][m][n]
    float *y;             // [m][ldy]
    uint32_t m, n, ldy, ksplit;
    uint32_t elem; // element type of y
};

struct GatherParams {
    const uint8_t *table;   // [vocab] rows of row_bytes
    const uint32_t *ids;    // [count]
    float *out;             // [count][hidden]
    uint32_t vocab, hidden, row_bytes;
    uint32_t quads_per_row; // hidden / 4
    uint32_t count;
    float scale;            // 1.0f when the lookup is not scaled
    uint32_t elem;          // the 16-bit kernels: element type of out (ELEM_F16 / ELEM_BF16)
};

struct GluActParams {
    const float *g; // gate results, row r at g + r * ld
    const float *u; // up results, row r at u + r * ld
    float *h;       // [m][ffn]
    uint32_t m, ffn, ld, relu_gate;
};

struct ConvertParams {
    const void *src;
    void *dst;
    uint64_t count;  // elements
    uint32_t elem;   // the 16-bit type (ELEM_F16 / ELEM_BF16); gq_finish_elem: any element type
    uint32_t widen;  // 1: 16-bit -> f32, 0: f32 -> 16-bit
    uint32_t accumulate, pad; // gq_finish_elem: dst = round(dst + src) instead of round(src)
};

struct ArgmaxParams {
    const float *logits; // [rows][ld]
    uint32_t *token;     // [rows]
    float *value;        // [rows] or null: the winning logit
    uint64_t *keys;      // [rows][parts] scratch between the two launches
    uint32_t n, ld;      // entries per row, elements between rows
    uint32_t parts;      // workgroups per row
    uint32_t chunk;      // entries per part
};

constexpr uint32_t ARGMAX_NONE = 0xFFFFFFFFu; // the row has no entry that is not NaN
constexpr uint32_t ARGMAX_MAX_PARTS = 128, ARGMAX_MAX_ROWS = 64; // scratch keys per launch pair

struct MoeJob {
    uint32_t expert;
    uint32_t p0;     // sorted position of the job's first pair
    uint32_t m;      // pairs in the job: 1 or 2
    uint32_t t0, t1; // their tokens (t1 = t0 when m = 1)
};

// All tokens of one expert, up to eight (or four) at a time: a job of the int8 matrix-core kernels.
struct MoeJob8 {
    uint32_t expert;
    uint32_t p0;     // sorted position of the job's first pair
    uint32_t m;      // pairs in the job: 1..8
    uint32_t pad;
    uint32_t tok[8]; // their tokens (entries past m repeat the last one)
};

struct MoePlanParams {
    const uint32_t *route_expert; // [tokens][top_k]
    const uint32_t *route_len;    // [tokens]
    uint32_t *pair_src;
    uint32_t *pair_pos;
    MoeJob *jobs;
    MoeJob8 *jobs8;   // written when P.fast
    uint32_t *counters; // [0] jobs, [1] routed pairs, [2] eight-token jobs
    uint32_t tokens, top_k, experts, pairs;
    uint32_t fast; // pairs are few enough for the per-pair placement (LDS has two more arrays of `pairs` words)
    uint32_t job_shift; // a matrix-core job takes up to 1 << job_shift tokens of an expert (3, or 2 for the streamed kernels)
};

constexpr uint32_t MOE_NONE = 0xFFFFFFFFu;

struct MoeGemvParams {
    GemvParams g;            // shape, split and LDS fields; w/x/y are the bases
    const MoeJob *jobs;
    const uint32_t *counters;
    uint64_t expert_stride;  // bytes between experts in g.w
    uint32_t wgs_per_job;
    uint32_t x_by_token;     // 1: activation row = token index, 0: sorted position
    uint32_t x_stride;       // elements between activation rows
    uint32_t y_stride;       // elements between output rows (by sorted position)
};

struct MoeMm8Params {
    Mm8Params g;             // shape of one expert's matrix; w, x, y are the bases
    const MoeJob8 *jobs;
    const uint32_t *counters;
    uint64_t expert_stride;  // bytes between experts in g.w
    const uint8_t *up;       // gated form: the up rows of expert 0 (g.w then holds the gate rows)
    uint64_t up_stride;      // bytes between experts in `up`
    uint32_t slices;         // workgroups that share one job's tiles (the streamed kernels cut runs of tiles across jobs instead)
    uint32_t y_stride;       // elements between output rows (by sorted position)
    const uint32_t *rows;    // null: the activation rows are the job's tokens; else this table (0, 1, ...)
                             // counts from the job's first sorted position
};

// Router (route.hip.inc): gate logits -> route table.
struct MoeRouteParams {
    const float *logits;     // [tokens][experts]
    uint32_t *route_expert;  // [tokens][top_k]
    float *route_weight;     // [tokens][top_k]
    uint32_t *route_len;     // [tokens]
    uint32_t *route_pos;     // [tokens][top_k] or null: the token's place in its expert's list
    uint32_t *expert_counts; // [experts] or null
    uint32_t *overflow;      // [1] or null: choices dropped because their expert was full
    uint32_t tokens, experts, top_k;
    uint32_t capacity;       // tokens an expert takes
    uint32_t phases;         // bit 0: softmax and top-k, bit 1: capacity filter (one workgroup)
};

constexpr int ROUTE_WAVES = 8;
constexpr int ROUTE_THREADS = 64 * ROUTE_WAVES;
constexpr uint32_t ROUTE_MAX_EXPERTS = 4096, ROUTE_MAX_TOP_K = 64;
constexpr uint32_t ROUTE_FUSED_MAX_TOKENS = 64; // up to here both phases are one launch

struct MoeActParams {
    const float *gu; // [pairs][2 * ffn]
    float *h;        // [pairs][ffn]
    const uint32_t *counters;
    uint32_t ffn, relu_gate;
};

struct MoeCombineParams {
    const float *o;               // [pairs][hidden] by sorted position
    const float *route_weight;    // [tokens][top_k]
    const uint32_t *route_len;    // [tokens]
    const uint32_t *pair_pos;     // [tokens][top_k]
    float *out;                   // [tokens][hidden]
    uint32_t tokens, top_k, hidden;
};

} // namespace gq

#endif
