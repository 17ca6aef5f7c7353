/*
 * CPU oracle (test infrastructure only, see gllmq_oracle.h for scope and pins).
 * Plain C11 + pthreads.  Build: make -C oracle   (-ffp-contract=off on purpose:
 * every product below is meant to be rounded exactly where the source says so).
 */
#include "gllmq_oracle.h"

#include <math.h>
#include <pthread.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256

/* ---------------------------------------------------------------- constants */
/* src/loader/gguf/types.rs:152-193 (block_size), :195-236 (block_bytes) */
size_t gq_block_size(uint32_t t)
{
    switch (t) {
    case GQ_TYPE_Q8_0: return 32;
    case GQ_TYPE_Q4_K:
    case GQ_TYPE_Q5_K:
    case GQ_TYPE_Q6_K: return QK_K;
    default: return 0;
    }
}

size_t gq_block_bytes(uint32_t t)
{
    switch (t) {
    case GQ_TYPE_Q8_0: return 34;
    case GQ_TYPE_Q4_K: return 144;
    case GQ_TYPE_Q5_K: return 176;
    case GQ_TYPE_Q6_K: return 210;
    default: return 0;
    }
}

/* src/loader/gguf/types.rs:443-472: the innermost dimension is padded to whole blocks */
size_t gq_row_bytes(uint32_t t, size_t k)
{
    size_t bs = gq_block_size(t);
    if (bs == 0) return 0;
    return ((k + bs - 1) / bs) * gq_block_bytes(t);
}

/* ------------------------------------------------------------ scalar helpers */
/* IEEE binary16 -> binary32, all classes (zero, subnormal, normal, inf, nan). */
float gq_f16_to_f32(uint16_t h)
{
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t expo = (h >> 10) & 0x1Fu;
    uint32_t mant = h & 0x3FFu;
    uint32_t bits;
    if (expo == 0) {
        if (mant == 0) {
            bits = sign;
        } else { /* subnormal: value = mant * 2^-24, renormalise */
            int shift = 0;
            while ((mant & 0x400u) == 0) { mant <<= 1; ++shift; }
            mant &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (mant << 13);
        }
    } else if (expo == 31) {
        bits = sign | 0x7F800000u | (mant << 13);
    } else {
        bits = sign | ((expo + (127 - 15)) << 23) | (mant << 13);
    }
    float f;
    memcpy(&f, &bits, sizeof f);
    return f;
}

/* half::bf16::from_f32 rounding (round to nearest, ties to even; NaN stays NaN),
 * the rule the reference applies when it narrows f32, src/compat/weight_helpers.rs:362-368 */
uint16_t gq_f32_to_bf16_rne(float f)
{
    uint32_t u;
    memcpy(&u, &f, sizeof u);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t round = 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)((u + round) >> 16);
}

static float bf16_round(float f)
{
    uint32_t u = (uint32_t)gq_f32_to_bf16_rne(f) << 16;
    float r;
    memcpy(&r, &u, sizeof r);
    return r;
}

static uint16_t rd16(const uint8_t *p) { return (uint16_t)(p[0] | (p[1] << 8)); }

/* quant-kquant-iq-proprietary.md:45-50 (get_scale_min_k4) */
void gq_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *m)
{
    if (j < 4) {
        *sc = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0F) | ((q[j - 4] >> 6) << 4));
        *m = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* ------------------------------------------------------------------- codecs */
/* Q4_K, 144 B: d f16 @0, dmin f16 @2, scales[12] @4, qs[128] @16.
 * quant-kquant-iq-proprietary.md:52-64,109-114: per 64-element group the low
 * nibbles are the first 32 elements, the high nibbles the next 32; min is subtracted. */
void gq_dequant_block_q4_k(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk));
    const float dmin = gq_f16_to_f32(rd16(blk + 2));
    const uint8_t *scales = blk + 4;
    const uint8_t *qs = blk + 16;
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, scales, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, scales, &sc1, &m1);
        const float d0 = d * (float)sc0, n0 = dmin * (float)m0;
        const float d1 = d * (float)sc1, n1 = dmin * (float)m1;
        const uint8_t *q = qs + 32 * g;
        float *o = out + 64 * g;
        for (int l = 0; l < 32; ++l) o[l] = d0 * (float)(q[l] & 0x0F) - n0;
        for (int l = 0; l < 32; ++l) o[32 + l] = d1 * (float)(q[l] >> 4) - n1;
    }
}

/* Q5_K, 176 B: d @0, dmin @2, scales[12] @4, qh[32] @16, qs[128] @48.
 * quant-kquant-iq-proprietary.md:145-154; tests/test_diag_q5km_block_bytes.rs:13-39:
 * fifth bit of element i is bit (i/32) of qh[i%32]. */
void gq_dequant_block_q5_k(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk));
    const float dmin = gq_f16_to_f32(rd16(blk + 2));
    const uint8_t *scales = blk + 4;
    const uint8_t *qh = blk + 16;
    const uint8_t *qs = blk + 48;
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, scales, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, scales, &sc1, &m1);
        const float d0 = d * (float)sc0, n0 = dmin * (float)m0;
        const float d1 = d * (float)sc1, n1 = dmin * (float)m1;
        const uint8_t *q = qs + 32 * g;
        float *o = out + 64 * g;
        for (int l = 0; l < 32; ++l) {
            int lo = (q[l] & 0x0F) + (((qh[l] >> (2 * g)) & 1) << 4);
            int hi = (q[l] >> 4) + (((qh[l] >> (2 * g + 1)) & 1) << 4);
            o[l] = d0 * (float)lo - n0;
            o[32 + l] = d1 * (float)hi - n1;
        }
    }
}

/* Q6_K, 210 B: ql[128] @0, qh[64] @128, scales i8[16] @192, d f16 @208.
 * quant-kquant-iq-proprietary.md:123-130; BUG-KNOWLEDGE.md:4021-4022,4121:
 * the four 2-bit fields of one qh byte belong to elements 32 apart. */
void gq_dequant_block_q6_k(const uint8_t *blk, float *out)
{
    const uint8_t *ql = blk;
    const uint8_t *qh = blk + 128;
    const int8_t *sc = (const int8_t *)(blk + 192);
    const float d = gq_f16_to_f32(rd16(blk + 208));
    for (int h = 0; h < 2; ++h) {
        for (int l = 0; l < 32; ++l) {
            const int is = 8 * h + l / 16;
            const uint8_t hb = qh[32 * h + l];
            const int q1 = (int)((ql[64 * h + l] & 0x0F) | (((hb >> 0) & 3) << 4)) - 32;
            const int q2 = (int)((ql[64 * h + 32 + l] & 0x0F) | (((hb >> 2) & 3) << 4)) - 32;
            const int q3 = (int)((ql[64 * h + l] >> 4) | (((hb >> 4) & 3) << 4)) - 32;
            const int q4 = (int)((ql[64 * h + 32 + l] >> 4) | (((hb >> 6) & 3) << 4)) - 32;
            float *o = out + 128 * h + l;
            o[0] = d * (float)sc[is + 0] * (float)q1;
            o[32] = d * (float)sc[is + 2] * (float)q2;
            o[64] = d * (float)sc[is + 4] * (float)q3;
            o[96] = d * (float)sc[is + 6] * (float)q4;
        }
    }
}

/* Q8_0, 34 B: d f16 @0, qs i8[32] @2.  gguf-classic-quant-layout.md:33,46 */
void gq_dequant_block_q8_0(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk));
    const int8_t *qs = (const int8_t *)(blk + 2);
    for (int i = 0; i < 32; ++i) out[i] = d * (float)qs[i];
}

typedef void (*block_fn)(const uint8_t *, float *);

static block_fn codec_for(uint32_t t)
{
    switch (t) {
    case GQ_TYPE_Q4_K: return gq_dequant_block_q4_k;
    case GQ_TYPE_Q5_K: return gq_dequant_block_q5_k;
    case GQ_TYPE_Q6_K: return gq_dequant_block_q6_k;
    case GQ_TYPE_Q8_0: return gq_dequant_block_q8_0;
    default: return NULL;
    }
}

/* src/compat/cpu_backend.rs:1066-1075: chunks_exact(block_bytes) zipped with
 * chunks_exact_mut(block_size); the shorter side ends the walk. */
int gq_dequantize(const uint8_t *blocks, size_t n_bytes, float *out, size_t n_out, uint32_t t)
{
    block_fn f = codec_for(t);
    if (!f) return GQ_ERR_UNIMPLEMENTED;
    const size_t bb = gq_block_bytes(t), bs = gq_block_size(t);
    size_t nb = n_bytes / bb;
    if (n_out / bs < nb) nb = n_out / bs;
    for (size_t b = 0; b < nb; ++b) f(blocks + b * bb, out + b * bs);
    return GQ_OK;
}

/* Op::QuantGather (src/arch/auto_graph_fragments/build_graph.inc.rs:203-211): row ids[i] of a
 * quantized table, decoded, times the embedding scale when there is one (`scaled`).  The op is
 * executed by generated code of gllm-kernels, which is not in the reference tree: that the scale
 * multiplies the decoded f32 value (one rounding) is this restatement's reading of
 * `Op::QuantGather { scale: Option<f32> }`; PARITY UNPINNED for scaled lookups.  An id outside
 * the table is an error here. */
int gq_quant_gather(const uint8_t *table, uint32_t t, size_t vocab, size_t hidden, const uint32_t *ids,
                    size_t count, float scale, int scaled, float *out)
{
    block_fn f = codec_for(t);
    if (!f) return GQ_ERR_UNIMPLEMENTED;
    const size_t bb = gq_block_bytes(t), bs = gq_block_size(t), rb = gq_row_bytes(t, hidden);
    float tmp[256];
    for (size_t i = 0; i < count; ++i) {
        if (ids[i] >= vocab) return GQ_ERR_BAD_SHAPE;
        const uint8_t *row = table + (size_t)ids[i] * rb;
        for (size_t e0 = 0, b = 0; e0 < hidden; e0 += bs, ++b) {
            f(row + b * bb, tmp);
            const size_t n = hidden - e0 < bs ? hidden - e0 : bs;
            for (size_t e = 0; e < n; ++e) out[i * hidden + e0 + e] = scaled ? tmp[e] * scale : tmp[e];
        }
    }
    return GQ_OK;
}

/* argmax_token, src/engine/executor_step.rs:48-55: entries that are NaN are filtered out, then
 * Iterator::max_by(partial_cmp), which keeps the LAST of several equal maxima (-0.0 == +0.0).
 * Returns -1 for the reference's None (empty or all NaN). */
int64_t gq_argmax_token(const float *logits, size_t n)
{
    int64_t best = -1;
    for (size_t i = 0; i < n; ++i) {
        if (logits[i] != logits[i]) continue;
        if (best < 0 || !(logits[i] < logits[best])) best = (int64_t)i; /* >= : a later equal entry replaces */
    }
    return best;
}

/* ------------------------------------------------- vectorised flavour (AVX2) */
/* The same decoders eight elements at a time, and a dot product over eight-lane partial sums:
 * the "AVX2 / AVX-512" side of the CPU baseline.  Every decoded value equals the scalar
 * decoder's bit for bit (the products d*sc*q are exact in f32, so a fused multiply-subtract
 * rounds like the scalar multiply then subtract); only the summation order of the dot product
 * differs from GQ_ACC_F32. */
#if defined(__AVX2__) && defined(__FMA__)
#include <immintrin.h>
#define GQ_HAVE_AVX2 1

static inline __m256 u8x8_to_ps(__m128i bytes) { return _mm256_cvtepi32_ps(_mm256_cvtepu8_epi32(bytes)); }

static void dequant_block_q4_k_avx2(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk)), dmin = gq_f16_to_f32(rd16(blk + 2));
    const __m128i low4 = _mm_set1_epi8(0x0F);
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, blk + 4, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, blk + 4, &sc1, &m1);
        const __m256 d0 = _mm256_set1_ps(d * (float)sc0), n0 = _mm256_set1_ps(dmin * (float)m0);
        const __m256 d1 = _mm256_set1_ps(d * (float)sc1), n1 = _mm256_set1_ps(dmin * (float)m1);
        for (int l = 0; l < 32; l += 8) {
            const __m128i q = _mm_loadl_epi64((const __m128i *)(blk + 16 + 32 * g + l));
            const __m128i lo = _mm_and_si128(q, low4), hi = _mm_and_si128(_mm_srli_epi16(q, 4), low4);
            _mm256_storeu_ps(out + 64 * g + l, _mm256_fmsub_ps(d0, u8x8_to_ps(lo), n0));
            _mm256_storeu_ps(out + 64 * g + 32 + l, _mm256_fmsub_ps(d1, u8x8_to_ps(hi), n1));
        }
    }
}

static void dequant_block_q5_k_avx2(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk)), dmin = gq_f16_to_f32(rd16(blk + 2));
    const __m128i low4 = _mm_set1_epi8(0x0F), one = _mm_set1_epi8(1);
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, blk + 4, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, blk + 4, &sc1, &m1);
        const __m256 d0 = _mm256_set1_ps(d * (float)sc0), n0 = _mm256_set1_ps(dmin * (float)m0);
        const __m256 d1 = _mm256_set1_ps(d * (float)sc1), n1 = _mm256_set1_ps(dmin * (float)m1);
        for (int l = 0; l < 32; l += 8) {
            const __m128i q = _mm_loadl_epi64((const __m128i *)(blk + 48 + 32 * g + l));
            const __m128i qh = _mm_loadl_epi64((const __m128i *)(blk + 16 + l));
            /* bit 2g of qh is the fifth bit of the low-nibble element, bit 2g+1 of the high one */
            const __m128i b0 = _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(qh, 2 * g), one), 4);
            const __m128i b1 = _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(qh, 2 * g + 1), one), 4);
            const __m128i lo = _mm_or_si128(_mm_and_si128(q, low4), b0);
            const __m128i hi = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(q, 4), low4), b1);
            _mm256_storeu_ps(out + 64 * g + l, _mm256_fmsub_ps(d0, u8x8_to_ps(lo), n0));
            _mm256_storeu_ps(out + 64 * g + 32 + l, _mm256_fmsub_ps(d1, u8x8_to_ps(hi), n1));
        }
    }
}

static void dequant_block_q6_k_avx2(const uint8_t *blk, float *out)
{
    const int8_t *sc = (const int8_t *)(blk + 192);
    const float d = gq_f16_to_f32(rd16(blk + 208));
    const __m128i low4 = _mm_set1_epi8(0x0F), two = _mm_set1_epi8(3);
    const __m256 off = _mm256_set1_ps(32.0f);
    for (int h = 0; h < 2; ++h)
        for (int l = 0; l < 32; l += 8) {
            const int is = 8 * h + l / 16;
            const __m128i a = _mm_loadl_epi64((const __m128i *)(blk + 64 * h + l));
            const __m128i b = _mm_loadl_epi64((const __m128i *)(blk + 64 * h + 32 + l));
            const __m128i hb = _mm_loadl_epi64((const __m128i *)(blk + 128 + 32 * h + l));
            const __m128i q1 = _mm_or_si128(_mm_and_si128(a, low4), _mm_slli_epi16(_mm_and_si128(hb, two), 4));
            const __m128i q2 = _mm_or_si128(_mm_and_si128(b, low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 2), two), 4));
            const __m128i q3 = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(a, 4), low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 4), two), 4));
            const __m128i q4 = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(b, 4), low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 6), two), 4));
            /* d * sc * (q - 32): q - 32 is exact, both products are exact in f32 */
            float *o = out + 128 * h + l;
            _mm256_storeu_ps(o, _mm256_mul_ps(_mm256_set1_ps(d * (float)sc[is + 0]), _mm256_sub_ps(u8x8_to_ps(q1), off)));
            _mm256_storeu_ps(o + 32, _mm256_mul_ps(_mm256_set1_ps(d * (float)sc[is + 2]), _mm256_sub_ps(u8x8_to_ps(q2), off)));
            _mm256_storeu_ps(o + 64, _mm256_mul_ps(_mm256_set1_ps(d * (float)sc[is + 4]), _mm256_sub_ps(u8x8_to_ps(q3), off)));
            _mm256_storeu_ps(o + 96, _mm256_mul_ps(_mm256_set1_ps(d * (float)sc[is + 6]), _mm256_sub_ps(u8x8_to_ps(q4), off)));
        }
}

static void dequant_block_q8_0_avx2(const uint8_t *blk, float *out)
{
    const __m256 d = _mm256_set1_ps(gq_f16_to_f32(rd16(blk)));
    for (int i = 0; i < 32; i += 8) {
        const __m128i q = _mm_loadl_epi64((const __m128i *)(blk + 2 + i));
        _mm256_storeu_ps(out + i, _mm256_mul_ps(d, _mm256_cvtepi32_ps(_mm256_cvtepi8_epi32(q))));
    }
}

/* sum of w[e] * x[e], e < len: four eight-lane partial sums over whole groups of 32, the lanes
 * added pairwise at the end, the tail one element at a time */
static float dot_avx2(const float *w, const float *x, size_t len, float carry)
{
    __m256 a0 = _mm256_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    size_t e = 0;
    for (; e + 32 <= len; e += 32) {
        a0 = _mm256_fmadd_ps(_mm256_loadu_ps(w + e), _mm256_loadu_ps(x + e), a0);
        a1 = _mm256_fmadd_ps(_mm256_loadu_ps(w + e + 8), _mm256_loadu_ps(x + e + 8), a1);
        a2 = _mm256_fmadd_ps(_mm256_loadu_ps(w + e + 16), _mm256_loadu_ps(x + e + 16), a2);
        a3 = _mm256_fmadd_ps(_mm256_loadu_ps(w + e + 24), _mm256_loadu_ps(x + e + 24), a3);
    }
    const __m256 s = _mm256_add_ps(_mm256_add_ps(a0, a1), _mm256_add_ps(a2, a3));
    __m128 q = _mm_add_ps(_mm256_castps256_ps128(s), _mm256_extractf128_ps(s, 1));
    q = _mm_add_ps(q, _mm_movehl_ps(q, q));
    q = _mm_add_ss(q, _mm_shuffle_ps(q, q, 1));
    float sum = carry + _mm_cvtss_f32(q);
    for (; e < len; ++e) sum += w[e] * x[e];
    return sum;
}

static block_fn codec_avx2_for(uint32_t t)
{
    switch (t) {
    case GQ_TYPE_Q4_K: return dequant_block_q4_k_avx2;
    case GQ_TYPE_Q5_K: return dequant_block_q5_k_avx2;
    case GQ_TYPE_Q6_K: return dequant_block_q6_k_avx2;
    case GQ_TYPE_Q8_0: return dequant_block_q8_0_avx2;
    default: return NULL;
    }
}
#else
#define GQ_HAVE_AVX2 0
#endif

/* ----------------------------------------------- vectorised flavour (AVX-512) */
/* The same again sixteen elements at a time, compiled for AVX-512 F/BW/VL by function attribute
 * (the file's baseline is x86-64-v3) and chosen at run time where the host has them.  Decoded
 * values equal the scalar decoder's bit for bit, for the reasons given above. */
#if GQ_HAVE_AVX2 && defined(__GNUC__)
#define GQ_HAVE_AVX512 1
#define GQ_T512 __attribute__((target("avx512f,avx512bw,avx512vl,avx512dq,fma")))

GQ_T512 static inline __m512 u8x16_to_ps(__m128i bytes) { return _mm512_cvtepi32_ps(_mm512_cvtepu8_epi32(bytes)); }

GQ_T512 static void dequant_block_q4_k_avx512(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk)), dmin = gq_f16_to_f32(rd16(blk + 2));
    const __m128i low4 = _mm_set1_epi8(0x0F);
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, blk + 4, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, blk + 4, &sc1, &m1);
        const __m512 d0 = _mm512_set1_ps(d * (float)sc0), n0 = _mm512_set1_ps(dmin * (float)m0);
        const __m512 d1 = _mm512_set1_ps(d * (float)sc1), n1 = _mm512_set1_ps(dmin * (float)m1);
        for (int l = 0; l < 32; l += 16) {
            const __m128i q = _mm_loadu_si128((const __m128i *)(blk + 16 + 32 * g + l));
            const __m128i lo = _mm_and_si128(q, low4), hi = _mm_and_si128(_mm_srli_epi16(q, 4), low4);
            _mm512_storeu_ps(out + 64 * g + l, _mm512_fmsub_ps(d0, u8x16_to_ps(lo), n0));
            _mm512_storeu_ps(out + 64 * g + 32 + l, _mm512_fmsub_ps(d1, u8x16_to_ps(hi), n1));
        }
    }
}

GQ_T512 static void dequant_block_q5_k_avx512(const uint8_t *blk, float *out)
{
    const float d = gq_f16_to_f32(rd16(blk)), dmin = gq_f16_to_f32(rd16(blk + 2));
    const __m128i low4 = _mm_set1_epi8(0x0F), one = _mm_set1_epi8(1);
    for (int g = 0; g < 4; ++g) {
        uint8_t sc0, m0, sc1, m1;
        gq_scale_min_k4(2 * g, blk + 4, &sc0, &m0);
        gq_scale_min_k4(2 * g + 1, blk + 4, &sc1, &m1);
        const __m512 d0 = _mm512_set1_ps(d * (float)sc0), n0 = _mm512_set1_ps(dmin * (float)m0);
        const __m512 d1 = _mm512_set1_ps(d * (float)sc1), n1 = _mm512_set1_ps(dmin * (float)m1);
        for (int l = 0; l < 32; l += 16) {
            const __m128i q = _mm_loadu_si128((const __m128i *)(blk + 48 + 32 * g + l));
            const __m128i qh = _mm_loadu_si128((const __m128i *)(blk + 16 + l));
            const __m128i b0 = _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(qh, 2 * g), one), 4);
            const __m128i b1 = _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(qh, 2 * g + 1), one), 4);
            const __m128i lo = _mm_or_si128(_mm_and_si128(q, low4), b0);
            const __m128i hi = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(q, 4), low4), b1);
            _mm512_storeu_ps(out + 64 * g + l, _mm512_fmsub_ps(d0, u8x16_to_ps(lo), n0));
            _mm512_storeu_ps(out + 64 * g + 32 + l, _mm512_fmsub_ps(d1, u8x16_to_ps(hi), n1));
        }
    }
}

GQ_T512 static void dequant_block_q6_k_avx512(const uint8_t *blk, float *out)
{
    const int8_t *sc = (const int8_t *)(blk + 192);
    const float d = gq_f16_to_f32(rd16(blk + 208));
    const __m128i low4 = _mm_set1_epi8(0x0F), two = _mm_set1_epi8(3);
    const __m512 off = _mm512_set1_ps(32.0f);
    for (int h = 0; h < 2; ++h)
        for (int l = 0; l < 32; l += 16) { /* sixteen elements share one scale */
            const int is = 8 * h + l / 16;
            const __m128i a = _mm_loadu_si128((const __m128i *)(blk + 64 * h + l));
            const __m128i b = _mm_loadu_si128((const __m128i *)(blk + 64 * h + 32 + l));
            const __m128i hb = _mm_loadu_si128((const __m128i *)(blk + 128 + 32 * h + l));
            const __m128i q1 = _mm_or_si128(_mm_and_si128(a, low4), _mm_slli_epi16(_mm_and_si128(hb, two), 4));
            const __m128i q2 = _mm_or_si128(_mm_and_si128(b, low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 2), two), 4));
            const __m128i q3 = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(a, 4), low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 4), two), 4));
            const __m128i q4 = _mm_or_si128(_mm_and_si128(_mm_srli_epi16(b, 4), low4), _mm_slli_epi16(_mm_and_si128(_mm_srli_epi16(hb, 6), two), 4));
            float *o = out + 128 * h + l;
            _mm512_storeu_ps(o, _mm512_mul_ps(_mm512_set1_ps(d * (float)sc[is + 0]), _mm512_sub_ps(u8x16_to_ps(q1), off)));
            _mm512_storeu_ps(o + 32, _mm512_mul_ps(_mm512_set1_ps(d * (float)sc[is + 2]), _mm512_sub_ps(u8x16_to_ps(q2), off)));
            _mm512_storeu_ps(o + 64, _mm512_mul_ps(_mm512_set1_ps(d * (float)sc[is + 4]), _mm512_sub_ps(u8x16_to_ps(q3), off)));
            _mm512_storeu_ps(o + 96, _mm512_mul_ps(_mm512_set1_ps(d * (float)sc[is + 6]), _mm512_sub_ps(u8x16_to_ps(q4), off)));
        }
}

GQ_T512 static void dequant_block_q8_0_avx512(const uint8_t *blk, float *out)
{
    const __m512 d = _mm512_set1_ps(gq_f16_to_f32(rd16(blk)));
    for (int i = 0; i < 32; i += 16) {
        const __m128i q = _mm_loadu_si128((const __m128i *)(blk + 2 + i));
        _mm512_storeu_ps(out + i, _mm512_mul_ps(d, _mm512_cvtepi32_ps(_mm512_cvtepi8_epi32(q))));
    }
}

/* sum of w[e] * x[e], e < len: four sixteen-lane partial sums over whole groups of 64, the lanes
 * added up at the end, then single vectors, the tail one element at a time */
GQ_T512 static float dot_avx512(const float *w, const float *x, size_t len, float carry)
{
    __m512 a0 = _mm512_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    size_t e = 0;
    for (; e + 64 <= len; e += 64) {
        a0 = _mm512_fmadd_ps(_mm512_loadu_ps(w + e), _mm512_loadu_ps(x + e), a0);
        a1 = _mm512_fmadd_ps(_mm512_loadu_ps(w + e + 16), _mm512_loadu_ps(x + e + 16), a1);
        a2 = _mm512_fmadd_ps(_mm512_loadu_ps(w + e + 32), _mm512_loadu_ps(x + e + 32), a2);
        a3 = _mm512_fmadd_ps(_mm512_loadu_ps(w + e + 48), _mm512_loadu_ps(x + e + 48), a3);
    }
    for (; e + 16 <= len; e += 16) /* short blocks (Q8_0: 32 elements) and the last whole vectors */
        a0 = _mm512_fmadd_ps(_mm512_loadu_ps(w + e), _mm512_loadu_ps(x + e), a0);
    float sum = carry + _mm512_reduce_add_ps(_mm512_add_ps(_mm512_add_ps(a0, a1), _mm512_add_ps(a2, a3)));
    for (; e < len; ++e) sum += w[e] * x[e];
    return sum;
}

static block_fn codec_avx512_for(uint32_t t)
{
    switch (t) {
    case GQ_TYPE_Q4_K: return dequant_block_q4_k_avx512;
    case GQ_TYPE_Q5_K: return dequant_block_q5_k_avx512;
    case GQ_TYPE_Q6_K: return dequant_block_q6_k_avx512;
    case GQ_TYPE_Q8_0: return dequant_block_q8_0_avx512;
    default: return NULL;
    }
}
#else
#define GQ_HAVE_AVX512 0
#endif

int gq_have_avx512(void)
{
#if GQ_HAVE_AVX512
    return __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") && __builtin_cpu_supports("avx512vl") &&
           __builtin_cpu_supports("avx512dq");
#else
    return 0;
#endif
}

int gq_dequant_block_avx512(uint32_t t, const uint8_t *blk, float *out)
{
#if GQ_HAVE_AVX512
    block_fn f = codec_avx512_for(t);
    if (!f || !gq_have_avx512()) return GQ_ERR_UNIMPLEMENTED;
    f(blk, out);
    return GQ_OK;
#else
    (void)t; (void)blk; (void)out;
    return GQ_ERR_UNIMPLEMENTED;
#endif
}

int gq_have_avx2(void)
{
#if GQ_HAVE_AVX2
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
#else
    return 0;
#endif
}

int gq_dequant_block_avx2(uint32_t t, const uint8_t *blk, float *out)
{
#if GQ_HAVE_AVX2
    block_fn f = codec_avx2_for(t);
    if (!f || !gq_have_avx2()) return GQ_ERR_UNIMPLEMENTED;
    f(blk, out);
    return GQ_OK;
#else
    (void)t; (void)blk; (void)out;
    return GQ_ERR_UNIMPLEMENTED;
#endif
}

/* ------------------------------------------------------------------- matmul */
typedef struct {
    const uint8_t *w;
    const float *x;
    float *y;
    uint32_t t;
    size_t m, n, k;
    int mode; /* GQ_ACC_F32, GQ_ACC_F64, 2 = bf16 operands + f64 sum, 3 / 4 = AVX2 / AVX-512 decode and f32 dot */
    size_t row0, row1;
} mm_job;

static void *mm_worker(void *arg)
{
    const mm_job *j = (const mm_job *)arg;
    block_fn f = codec_for(j->t);
#if GQ_HAVE_AVX2
    if (j->mode == 3) f = codec_avx2_for(j->t);
#endif
#if GQ_HAVE_AVX512
    if (j->mode == 4) f = codec_avx512_for(j->t);
#endif
    const size_t bs = gq_block_size(j->t), bb = gq_block_bytes(j->t);
    const size_t nblk = (j->k + bs - 1) / bs;
    const size_t stride = nblk * bb;
    float tmp[QK_K];
    float *accf = (float *)malloc(j->m * sizeof(float));
    double *accd = (double *)malloc(j->m * sizeof(double));
    for (size_t r = j->row0; r < j->row1; ++r) {
        const uint8_t *row = j->w + r * stride;
        for (size_t i = 0; i < j->m; ++i) { accf[i] = 0.0f; accd[i] = 0.0; }
        for (size_t b = 0; b < nblk; ++b) {
            f(row + b * bb, tmp);
            const size_t k0 = b * bs;
            const size_t len = (k0 + bs <= j->k) ? bs : j->k - k0; /* row padding is dropped */
            if (j->mode == 2)
                for (size_t e = 0; e < len; ++e) tmp[e] = bf16_round(tmp[e]);
            for (size_t i = 0; i < j->m; ++i) {
                const float *xi = j->x + i * j->k + k0;
#if GQ_HAVE_AVX2
                if (j->mode == 3) {
                    accf[i] = dot_avx2(tmp, xi, len, accf[i]);
                    continue;
                }
#endif
#if GQ_HAVE_AVX512
                if (j->mode == 4) {
                    accf[i] = dot_avx512(tmp, xi, len, accf[i]);
                    continue;
                }
#endif
                if (j->mode == GQ_ACC_F32) {
                    float a = accf[i];
                    for (size_t e = 0; e < len; ++e) a += tmp[e] * xi[e];
                    accf[i] = a;
                } else if (j->mode == GQ_ACC_F64) {
                    double a = accd[i];
                    for (size_t e = 0; e < len; ++e) a += (double)tmp[e] * (double)xi[e];
                    accd[i] = a;
                } else {
                    double a = accd[i];
                    for (size_t e = 0; e < len; ++e) a += (double)tmp[e] * (double)bf16_round(xi[e]);
                    accd[i] = a;
                }
            }
        }
        for (size_t i = 0; i < j->m; ++i)
            j->y[i * j->n + r] = (j->mode == GQ_ACC_F32 || j->mode == 3 || j->mode == 4) ? accf[i] : (float)accd[i];
    }
    free(accf);
    free(accd);
    return NULL;
}

static int mm_run(const uint8_t *w, const float *x, float *y, uint32_t t, size_t m, size_t n,
                  size_t k, int mode, int threads)
{
    if (!codec_for(t)) return GQ_ERR_UNIMPLEMENTED;
    if (m == 0 || n == 0) return GQ_OK;
    if (threads < 1) threads = 1;
    if ((size_t)threads > n) threads = (int)n;
    mm_job *jobs = (mm_job *)calloc((size_t)threads, sizeof(mm_job));
    pthread_t *tid = (pthread_t *)calloc((size_t)threads, sizeof(pthread_t));
    const size_t per = (n + (size_t)threads - 1) / (size_t)threads;
    int started = 0;
    for (int i = 0; i < threads; ++i) {
        size_t r0 = (size_t)i * per, r1 = r0 + per;
        if (r0 >= n) break;
        if (r1 > n) r1 = n;
        jobs[i] = (mm_job){ w, x, y, t, m, n, k, mode, r0, r1 };
        if (threads == 1) {
            mm_worker(&jobs[i]);
        } else {
            pthread_create(&tid[i], NULL, mm_worker, &jobs[i]);
            ++started;
        }
    }
    for (int i = 0; i < started; ++i) pthread_join(tid[i], NULL);
    free(jobs);
    free(tid);
    return GQ_OK;
}

/* src/compat/cpu_backend.rs:991-1049 */
int gq_quantized_matmul(const uint8_t *w, const float *x, float *y, uint32_t t, size_t m,
                        size_t n, size_t k, int acc_mode, int threads)
{
    if (acc_mode != GQ_ACC_F32 && acc_mode != GQ_ACC_F64) return GQ_ERR_BAD_SHAPE;
    return mm_run(w, x, y, t, m, n, k, acc_mode, threads);
}

int gq_quantized_matmul_bf16(const uint8_t *w, const float *x, float *y, uint32_t t, size_t m,
                             size_t n, size_t k, int threads)
{
    return mm_run(w, x, y, t, m, n, k, 2, threads);
}

int gq_quantized_matmul_avx2(const uint8_t *w, const float *x, float *y, uint32_t t, size_t m,
                             size_t n, size_t k, int threads)
{
    if (!gq_have_avx2()) return GQ_ERR_UNIMPLEMENTED;
    return mm_run(w, x, y, t, m, n, k, 3, threads);
}

int gq_quantized_matmul_avx512(const uint8_t *w, const float *x, float *y, uint32_t t, size_t m,
                               size_t n, size_t k, int threads)
{
    if (!gq_have_avx512()) return GQ_ERR_UNIMPLEMENTED;
    return mm_run(w, x, y, t, m, n, k, 4, threads);
}

/* ---------------------------------------------------------------------- MoE */
/* src/moe/routing.rs:290-302 */
void gq_softmax(const float *logits, size_t n, float *probs)
{
    if (n == 0) return;
    float mx = -INFINITY;
    for (size_t i = 0; i < n; ++i) mx = fmaxf(mx, logits[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; ++i) {
        probs[i] = expf(logits[i] - mx);
        sum += probs[i];
    }
    if (sum > 0.0f) {
        for (size_t i = 0; i < n; ++i) probs[i] = probs[i] / sum;
    } else {
        for (size_t i = 0; i < n; ++i) probs[i] = 1.0f / (float)n;
    }
}

/* Stable descending order on `key` (Rust's sort_by is stable; an unordered
 * comparison counts as equal, src/moe/routing.rs:268). */
static void stable_desc_order(const float *key, size_t n, uint32_t *order)
{
    for (size_t i = 0; i < n; ++i) {
        size_t p = i;
        while (p > 0 && key[order[p - 1]] < key[i]) {
            order[p] = order[p - 1];
            --p;
        }
        order[p] = (uint32_t)i;
    }
}

/* src/moe/routing.rs:263-280 */
size_t gq_topk_with_weights(const float *logits, size_t n, size_t k, uint32_t *idx, float *w)
{
    if (n == 0) return 0;
    float *p = (float *)malloc(n * sizeof(float));
    uint32_t *ord = (uint32_t *)malloc(n * sizeof(uint32_t));
    gq_softmax(logits, n, p);
    stable_desc_order(p, n, ord);
    const size_t kk = k < n ? k : n;
    float sum = 0.0f;
    for (size_t i = 0; i < kk; ++i) {
        idx[i] = ord[i];
        w[i] = p[ord[i]];
        sum += w[i];
    }
    if (sum > 0.0f)
        for (size_t i = 0; i < kk; ++i) w[i] /= sum;
    free(p);
    free(ord);
    return kk;
}

/* src/moe/routing.rs:283-287 */
size_t gq_topk_indices(const float *logits, size_t n, size_t k, uint32_t *idx)
{
    if (n == 0) return 0;
    uint32_t *ord = (uint32_t *)malloc(n * sizeof(uint32_t));
    stable_desc_order(logits, n, ord);
    const size_t kk = k < n ? k : n;
    for (size_t i = 0; i < kk; ++i) idx[i] = ord[i];
    free(ord);
    return kk;
}

/* src/moe/routing.rs:53-61 */
size_t gq_expert_capacity(float capacity_factor, size_t total_tokens, size_t num_experts)
{
    float v = ceilf(capacity_factor * (float)total_tokens / (float)num_experts);
    if (isnan(v) || v < 0.0f) return 0;
    if (v > 1.0e9f) v = 1.0e9f;
    return (size_t)v;
}

/* src/moe/routing.rs:100-160 */
size_t gq_route(const float *logits, size_t tokens, size_t experts, size_t top_k,
                float capacity_factor, uint32_t *route_expert, float *route_weight,
                uint32_t *route_pos, uint32_t *route_len, uint32_t *expert_counts)
{
    const size_t cap = gq_expert_capacity(capacity_factor, tokens, experts);
    const size_t stride = top_k ? top_k : 1; /* row length of the route arrays: a token always gets one slot */
    size_t overflow = 0;
    uint32_t *idx = (uint32_t *)malloc((top_k ? top_k : 1) * sizeof(uint32_t));
    float *w = (float *)malloc((top_k ? top_k : 1) * sizeof(float));
    for (size_t e = 0; e < experts; ++e) expert_counts[e] = 0;
    for (size_t t = 0; t < tokens; ++t) {
        const size_t kk = gq_topk_with_weights(logits + t * experts, experts, top_k, idx, w);
        uint32_t len = 0;
        for (size_t i = 0; i < kk; ++i) {
            const uint32_t e = idx[i];
            if (expert_counts[e] < cap) {
                route_expert[t * stride + len] = e;
                route_weight[t * stride + len] = w[i];
                route_pos[t * stride + len] = expert_counts[e];
                ++expert_counts[e];
                ++len;
            } else {
                ++overflow;
            }
        }
        if (len == 0 && experts > 0) { /* no choice kept (all full, or top_k = 0): least-loaded expert, weight 1 */
            size_t best = 0;
            for (size_t e = 1; e < experts; ++e)
                if (expert_counts[e] < expert_counts[best]) best = e;
            route_expert[t * stride] = (uint32_t)best;
            route_weight[t * stride] = 1.0f;
            route_pos[t * stride] = expert_counts[best];
            ++expert_counts[best];
            len = 1;
        }
        route_len[t] = len;
    }
    free(idx);
    free(w);
    return overflow;
}

static float silu(float g) { return g / (1.0f + expf(-g)); }

/* Expert FFN down(silu(gate x) * (up x)) (SPEC/MD-ARCHIVE/04-OPERATORS.md:114,146;
 * build_graph.inc.rs:2089-2117), combined as out += expert_out * weight in route
 * order (src/moe/routing.rs:307-327). */
int gq_moe_ffn(const uint8_t *gate_up, uint32_t t_gu, const uint8_t *down, uint32_t t_dn,
               const float *x, float *out, size_t tokens, size_t hidden, size_t ffn,
               size_t experts, size_t top_k, const uint32_t *route_expert,
               const float *route_weight, const uint32_t *route_len, int relu_gate,
               int acc_mode, int threads)
{
    if (!codec_for(t_gu) || !codec_for(t_dn)) return GQ_ERR_UNIMPLEMENTED;
    const size_t gu_bytes = 2 * ffn * gq_row_bytes(t_gu, hidden);
    const size_t dn_bytes = hidden * gq_row_bytes(t_dn, ffn);
    float *gu = (float *)malloc(2 * ffn * sizeof(float));
    float *h = (float *)malloc(ffn * sizeof(float));
    float *o = (float *)malloc(hidden * sizeof(float));
    for (size_t t = 0; t < tokens; ++t) {
        float *yt = out + t * hidden;
        for (size_t i = 0; i < hidden; ++i) yt[i] = 0.0f;
        for (uint32_t r = 0; r < route_len[t]; ++r) {
            const uint32_t e = route_expert[t * top_k + r];
            if (e >= experts) { free(gu); free(h); free(o); return GQ_ERR_BAD_SHAPE; }
            const float wgt = route_weight[t * top_k + r];
            mm_run(gate_up + (size_t)e * gu_bytes, x + t * hidden, gu, t_gu, 1, 2 * ffn, hidden,
                   acc_mode, threads);
            for (size_t i = 0; i < ffn; ++i) {
                float g = gu[i];
                if (relu_gate) g = g > 0.0f ? g : 0.0f;
                h[i] = silu(g) * gu[ffn + i];
            }
            mm_run(down + (size_t)e * dn_bytes, h, o, t_dn, 1, hidden, ffn, acc_mode, threads);
            for (size_t i = 0; i < hidden; ++i) yt[i] += o[i] * wgt;
        }
    }
    free(gu);
    free(h);
    free(o);
    return GQ_OK;
}

/* Dense feed-forward block (src/arch/auto_graph_fragments/build_graph.inc.rs:1957-1995): the
 * gate and up products, h = silu(gate) * up in f32 (Op::SwiGlu), the down product.  The
 * products are gq_quantized_matmul's (same accumulation modes). */
int gq_ffn_swiglu(const uint8_t *gate, const uint8_t *up, uint32_t t_gu, const uint8_t *down, uint32_t t_dn,
                  const float *x, float *out, size_t m, size_t hidden, size_t ffn, int relu_gate, int acc, int threads)
{
    float *g = (float *)malloc(sizeof(float) * m * ffn * 2);
    if (!g) return GQ_ERR_BAD_SHAPE;
    float *u = g + m * ffn;
    int rc = gq_quantized_matmul(gate, x, g, t_gu, m, ffn, hidden, acc, threads);
    if (rc == GQ_OK) rc = gq_quantized_matmul(up, x, u, t_gu, m, ffn, hidden, acc, threads);
    if (rc == GQ_OK) {
        for (size_t i = 0; i < m * ffn; ++i) {
            float gv = g[i];
            if (relu_gate && !(gv > 0.0f)) gv = 0.0f;
            g[i] = silu(gv) * u[i];
        }
        rc = gq_quantized_matmul(down, g, out, t_dn, m, hidden, ffn, acc, threads);
    }
    free(g);
    return rc;
}
