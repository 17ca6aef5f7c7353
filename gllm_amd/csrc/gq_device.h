// Device-side helpers shared by the gfx950 kernels: block geometry, f16 decode,
// the packed 6-bit scale/min fields of Q4_K/Q5_K and wave64 reductions.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gq {

constexpr int WAVE = 64;
constexpr int QK_K = 256;

// GgmlDType ids (reference: src/loader/gguf/types.rs:57-94)
constexpr uint32_t T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14;

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h)
{
    // v_cvt_f32_f16 is IEEE for every class, subnormals included (f16 denormals are
    // never flushed on this target).
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(h & 0xFFFFu)));
}

// f32 -> nearest bf16 (ties to even) -> f32; NaN passes through.  Same rule as
// half::bf16::from_f32, which the reference uses (src/compat/weight_helpers.rs:1202-1215).
__device__ __forceinline__ float round_to_bf16(float v)
{
    uint32_t b = __builtin_bit_cast(uint32_t, v);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return v;
    b += 0x7FFFu + ((b >> 16) & 1u);
    return __builtin_bit_cast(float, b & 0xFFFF0000u);
}

typedef uint32_t u4v __attribute__((ext_vector_type(4))); // plain 16-byte register quad

// Element types of activations and outputs at the boundary (Backend<E>, E in {f32, f16, bf16},
// src/compat/mod.rs:376-378).  16-bit elements widen exactly on the way in; results are rounded to
// the nearest element, ties to even, on the way out (half::f16 / half::bf16 ::from_f32, the
// conversions of src/compat/jit_helpers.rs:35-50), NaN stays NaN.
constexpr uint32_t ELEM_F32 = 0, ELEM_F16 = 1, ELEM_BF16 = 2;

__device__ __forceinline__ float elem16_to_f32(uint32_t bits, uint32_t elem)
{
    return elem == ELEM_F16 ? f16_bits_to_f32(bits) : __builtin_bit_cast(float, bits << 16);
}

__device__ __forceinline__ uint16_t f32_to_elem16(float v, uint32_t elem)
{
    if (elem == ELEM_F16) return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
    const uint32_t b = __builtin_bit_cast(uint32_t, v);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return static_cast<uint16_t>((b >> 16) | 0x0040u); // NaN, made quiet
    return static_cast<uint16_t>((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
}

// y[idx] of an output whose elements are of type `elem` (y is typed for the f32 case)
__device__ __forceinline__ void store_elem(float *y, size_t idx, float v, uint32_t elem)
{
    if (elem == ELEM_F32) y[idx] = v;
    else reinterpret_cast<uint16_t *>(y)[idx] = f32_to_elem16(v, elem);
}

// Eight consecutive activations from element `idx` on (16-byte aligned for f32 and for 16-bit
// elements alike: two quads or one).
__device__ __forceinline__ void load_elem8(const float *x, size_t idx, uint32_t elem, float (&v)[8])
{
    if (elem == ELEM_F32) {
        const float4 a = *reinterpret_cast<const float4 *>(x + idx);
        const float4 c = *reinterpret_cast<const float4 *>(x + idx + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = c.x; v[5] = c.y; v[6] = c.z; v[7] = c.w;
    } else {
        const uint4 t = *reinterpret_cast<const uint4 *>(reinterpret_cast<const uint16_t *>(x) + idx);
        const uint32_t w[4] = { t.x, t.y, t.z, t.w };
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = elem16_to_f32(w[i] & 0xFFFFu, elem);
            v[2 * i + 1] = elem16_to_f32(w[i] >> 16, elem);
        }
    }
}

// Candidates of the greedy token choice (argmax.hip.inc, and the GEMV that ends in it): the value
// mapped to an unsigned number of the same order above its index; 0 = no candidate (NaN).
__device__ __forceinline__ uint64_t argmax_key(float v, uint32_t idx)
{
    if (v != v) return 0ull;
    v += 0.0f; // -0.0 becomes +0.0: the two compare equal in the reference
    const uint32_t bits = __builtin_bit_cast(uint32_t, v);
    const uint32_t ord = (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
    return (static_cast<uint64_t>(ord) << 32) | idx;
}

__device__ __forceinline__ float argmax_key_value(uint64_t key)
{
    const uint32_t ord = static_cast<uint32_t>(key >> 32);
    const uint32_t bits = (ord & 0x80000000u) ? (ord & 0x7FFFFFFFu) : ~ord;
    return __builtin_bit_cast(float, bits);
}

// Block fixed point: the powers of two that turn a group of activations whose largest magnitude
// has the biased exponent `e_raw` (0 .. 254) into integers below 2^BITS and back.
//   |x| < 2^(e-126)   ->   |x * pre * up| < 2^BITS,   down = 1 / (pre * up) = 2^(e - 126 - BITS)
// With e >= BITS one multiplier does (pre = 1).  Smaller groups (down to subnormal ones, e = 1
// covers them) need more than 2^127: pre lifts the values first, exactly, and `down` is then a
// subnormal power of two, so such a group keeps its values to 2^(e-126-BITS) >= 2^-148 like any
// other instead of being rounded to multiples of 2^-126.
struct BlockScale {
    float pre, up, down;
};
template <int BITS>
__device__ __forceinline__ BlockScale block_scale(uint32_t e_raw)
{
    const uint32_t e = min(max(e_raw, 1u), 254u);
    const bool tiny = e < static_cast<uint32_t>(BITS);
    BlockScale s;
    s.pre = tiny ? __builtin_bit_cast(float, (static_cast<uint32_t>(BITS) + 126u - e) << 23) : 1.0f;
    s.up = tiny ? __builtin_bit_cast(float, 254u << 23) : __builtin_bit_cast(float, (static_cast<uint32_t>(BITS) + 253u - e) << 23);
    s.down = tiny ? __builtin_bit_cast(float, 1u << (e + 23u - static_cast<uint32_t>(BITS)))
                  : __builtin_bit_cast(float, (e + 1u - static_cast<uint32_t>(BITS)) << 23);
    return s;
}

// Loads of 2-byte aligned data as wider words.  gfx950 under the HSA ABI runs global
// memory in unaligned-access mode, so one load instruction serves any byte address.
template <typename T>
__device__ __forceinline__ T load_unaligned(const void *p)
{
    T v;
    __builtin_memcpy(&v, p, sizeof(T));
    return v;
}

// Gate activation of the feed-forward block: SiLU, behind a ReLU when `relu`
// (reference: Op::SwiGlu, silu(gate) * up, src/arch/auto_graph_fragments/build_graph.inc.rs:1977-1984).
// The hardware's exponential and reciprocal (about 1 ulp each): a kernel that applies the gate to
// the activations it loads does so in every workgroup, where a library exponential would cost
// microseconds.
__device__ __forceinline__ float glu_act(float g, bool relu)
{
    if (relu) g = g > 0.0f ? g : 0.0f;
    return g * __builtin_amdgcn_rcpf(1.0f + __expf(-g));
}

// (sc, m) pair j of the 12-byte field held as three little-endian dwords s0,s1,s2
// (bytes 0-3, 4-7, 8-11).  Reference: quant-kquant-iq-proprietary.md:45-50.
__device__ __forceinline__ void scale_min_k4(int j, uint32_t s0, uint32_t s1, uint32_t s2,
                                             uint32_t &sc, uint32_t &mn)
{
    const int sh = 8 * (j & 3);
    const uint32_t a = (s0 >> sh) & 0xFFu; // byte j&3 of scales[0..3]
    const uint32_t b = (s1 >> sh) & 0xFFu; // byte j&3 of scales[4..7]
    const uint32_t c = (s2 >> sh) & 0xFFu; // byte j&3 of scales[8..11]
    if (j < 4) {
        sc = a & 63u;
        mn = b & 63u;
    } else {
        sc = (c & 0xFu) | ((a >> 6) << 4);
        mn = (c >> 4) | ((b >> 6) << 4);
    }
}

// Byte n of a dword as f32 in one instruction.  Written as asm because the optimiser
// otherwise folds the caller's nibble mask into a bit-field extract per byte and spends
// two instructions where one does.
__device__ __forceinline__ float ubyte0(uint32_t v)
{
    float f;
    asm("v_cvt_f32_ubyte0 %0, %1" : "=v"(f) : "v"(v));
    return f;
}
__device__ __forceinline__ float ubyte1(uint32_t v)
{
    float f;
    asm("v_cvt_f32_ubyte1 %0, %1" : "=v"(f) : "v"(v));
    return f;
}
__device__ __forceinline__ float ubyte2(uint32_t v)
{
    float f;
    asm("v_cvt_f32_ubyte2 %0, %1" : "=v"(f) : "v"(v));
    return f;
}
__device__ __forceinline__ float ubyte3(uint32_t v)
{
    float f;
    asm("v_cvt_f32_ubyte3 %0, %1" : "=v"(f) : "v"(v));
    return f;
}

// Sum over a segment of `len` consecutive lanes (len a multiple of 4, segment start a
// multiple of 4, `pos` = lane's index inside its segment).  The total lands in the
// lane with pos == 0; other lanes hold partial garbage.
__device__ __forceinline__ float segment_sum(float v, int pos, int len)
{
    v += __shfl_xor(v, 1, WAVE);
    v += __shfl_xor(v, 2, WAVE);
#pragma unroll
    for (int off = 32; off >= 4; off >>= 1) {
        const float o = __shfl_down(v, off, WAVE);
        if (pos + off < len) v += o;
    }
    return v;
}

// Sum over all 64 lanes with DPP only (no LDS traffic); the total lands in lane 63.
template <int CTRL, int ROW_MASK, bool BOUND>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, BOUND));
}

__device__ __forceinline__ float wave_sum_to_last_lane(float v)
{
    v += dpp_f32<0x111, 0xF, true>(v); // row_shr:1
    v += dpp_f32<0x112, 0xF, true>(v); // row_shr:2
    v += dpp_f32<0x114, 0xF, true>(v); // row_shr:4
    v += dpp_f32<0x118, 0xF, true>(v); // row_shr:8  -> lane 15 of each row of 16 holds the row sum
    v += dpp_f32<0x142, 0xA, false>(v); // row_bcast:15 into rows 1 and 3
    v += dpp_f32<0x143, 0xC, false>(v); // row_bcast:31 into rows 2 and 3 -> lane 63 holds the total
    return v;
}

__device__ __forceinline__ float wave_sum(float v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

} // namespace gq
