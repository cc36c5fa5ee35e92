/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement ("oracle") of the arithmetic of
 * xorl's QLoRA weight codecs.  Nothing in the product package may import,
 * link or call this file; it exists so tests, the smoke check and the
 * benchmark's cpu_baseline leg have an independent answer to compare the HIP
 * kernels against.
 *
 * Every function cites the reference source (paths relative to the xorl
 * checkout) whose arithmetic it restates.  All float work is IEEE binary32,
 * one operation at a time (compile with -ffp-contract=off), because the
 * reference decode is "integer unpack, one or two fp32 multiplies/subtracts,
 * one round-to-nearest-even cast to bfloat16".
 *
 * Pin status (see tests/test_oracle_*.py):
 *   decode  int4 / nvfp4 / block_fp8 / nf4, flat and GKN .. pinned
 *       (exhaustive code enumeration vs torch.float8_e4m3fn / torch.bfloat16
 *        library casts, the e2m1 table, the reference-held block-fp8
 *        restatement, layout transposition identities, a numpy twin; nf4:
 *        the level table against the normal-quantile construction it is
 *        published with, decision points = fp32 mean of neighbouring levels)
 *   quantizers (int4 A2, nvfp4 A4, block_fp8 A6, nf4) ..... pinned for IEEE
 *        arithmetic; byte parity with a GPU-run Triton quantizer is UNPINNED
 *        (Triton's fp32 division / fma contraction / fp8 saturation are not
 *        fixed by the reference text).  Not required: oracle and kernels
 *        consume the same bytes.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define XQO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ */
/* scalar helpers                                                       */
/* ------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* fp32 -> bf16, round to nearest even; NaN stays NaN (quiet). */
XQO_API uint16_t xqo_bf16_rne(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

XQO_API float xqo_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* OCP e4m3fn byte -> fp32 (bias 7, no inf, 0x7f/0xff = NaN, max 448). */
XQO_API float xqo_e4m3_to_f32(uint8_t b) {
    uint32_t sign = (uint32_t)(b & 0x80u) << 24;
    uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
    if (e == 0xfu && m == 7u) return bits_f32(sign | 0x7fc00000u);
    float mag;
    if (e == 0) mag = (float)m * 0.001953125f;          /* m * 2^-9 */
    else mag = bits_f32(((e + 120u) << 23) | (m << 20)); /* 1.m * 2^(e-7) */
    return bits_f32(f32_bits(mag) | sign);
}

/* fp32 -> e4m3fn, round to nearest even, saturating to +-448 (the
 * "satfinite" behaviour of the reference's .to(tl.float8e4nv) on its target
 * hardware); NaN -> 0x7f|sign. */
XQO_API uint8_t xqo_f32_to_e4m3(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7fffffffu;
    if (a > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
    float af = bits_f32(a);
    if (af >= 448.0f) return (uint8_t)(sign | 0x7eu);
    if (af < 0.015625f) {                      /* below 2^-6: subnormal grid 2^-9 */
        float q = af * 512.0f;                 /* exact scaling */
        float r = nearbyintf(q);               /* RNE in default rounding mode */
        return (uint8_t)(sign | (uint8_t)r);   /* r in 0..8; 8 == 0x08 = 2^-6 */
    }
    /* normal: keep 3 mantissa bits */
    uint32_t lsb = (a >> 20) & 1u;
    a += 0x7ffffu + lsb;
    uint32_t e = (a >> 23) - 120u, m = (a >> 20) & 7u;
    uint32_t code = (e << 3) | m;
    if (code > 0x7eu) code = 0x7eu;
    return (uint8_t)(sign | code);
}

/* e2m1 nibble -> fp32.  Follows _fp4_decode, ops/quantize/fp4_codec.py:22-30:
 * magnitude code c = nib & 7, exponent field c >> 1, mantissa bit c & 1;
 * exponent 0 is the subnormal {0, 0.5}; sign is bit 3 (code 8 = -0.0). */
XQO_API float xqo_e2m1_to_f32(uint8_t nib) {
    uint32_t c = nib & 7u, e = c >> 1, m = c & 1u;
    uint32_t bits = e > 0 ? (((e + 126u) << 23) | (m << 22)) : m * 0x3f000000u;
    return bits_f32(bits | ((uint32_t)(nib & 8u) << 28));
}

/* fp32 -> e2m1 nibble.  Follows _fp4_encode, fp4_codec.py:12-19: linear codes
 * 0..3 by trunc(a*2+0.5) (ties up), log codes by thresholds 2.5/3.5/5.0,
 * switch at a >= 1.75; sign bit set for val < 0. */
XQO_API uint8_t xqo_f32_to_e2m1(float v) {
    uint8_t sign = v < 0.0f ? 8u : 0u;
    float a = fabsf(v);
    float t = a * 2.0f;
    t = t + 0.5f;
    int lo = (int)t;
    if (lo > 3) lo = 3;
    int hi = 4 + (a >= 2.5f) + (a >= 3.5f) + (a >= 5.0f);
    return (uint8_t)((a >= 1.75f ? hi : lo) + sign);
}

/* ------------------------------------------------------------------ */
/* int4                                                                 */
/* ------------------------------------------------------------------ */

/* flat [rows, cols], groups of `group` consecutive elements along cols.
 * Follows _int4_dequantize_kernel, ops/quantize/int4_quantize.py:45-76:
 * byte i holds element 2i in the low nibble and 2i+1 in the high nibble
 * (:62-63), w = bf16(fl(fl(nib - 8) * scale)) (:69-74); scales are fp32
 * (callers cast bf16 scales up first, :119). */
XQO_API void xqo_int4_decode_flat(const uint8_t* packed, const float* scales,
                                  uint16_t* out, int64_t n_elems, int64_t group) {
    for (int64_t i = 0; i < n_elems; ++i) {
        uint8_t b = packed[i >> 1];
        uint8_t nib = (i & 1) ? (b >> 4) : (b & 0xf);
        float d = (float)nib - 8.0f;
        float v = d * scales[i / group];
        out[i] = xqo_bf16_rne(v);
    }
}

/* GKN [K, N]: packed [K/2, N], byte (k2, n) holds K-rows 2*k2 (low) and
 * 2*k2+1 (high); scales [K/group, N].  Follows _int4_dequantize_gkn_kernel,
 * ops/quantize/int4_gkn_quantize.py:79-130. */
XQO_API void xqo_int4_decode_gkn(const uint8_t* packed, const float* scales,
                                 uint16_t* out, int64_t K, int64_t N, int64_t group) {
    for (int64_t k = 0; k < K; ++k)
        for (int64_t n = 0; n < N; ++n) {
            uint8_t b = packed[(k >> 1) * N + n];
            uint8_t nib = (k & 1) ? (b >> 4) : (b & 0xf);
            float d = (float)nib - 8.0f;
            float v = d * scales[(k / group) * N + n];
            out[k * N + n] = xqo_bf16_rne(v);
        }
}

/* Reference quantizer, _int4_quantize_kernel int4_quantize.py:12-41:
 * scale = max(amax, 1e-12) * (2/15); q = clamp(trunc(x * (1/scale) + 8.5), 0, 15). */
XQO_API void xqo_int4_quantize_flat(const float* x, uint8_t* packed, float* scales,
                                    int64_t n_elems, int64_t group) {
    const float two_fifteenths = (float)(2.0 / 15.0);
    for (int64_t g = 0; g < n_elems / group; ++g) {
        float amax = 0.0f;
        for (int64_t j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(x[g * group + j]));
        float scale = fmaxf(amax, 1e-12f) * two_fifteenths;
        scales[g] = scale;
        float inv = 1.0f / scale;
        for (int64_t j = 0; j < group; ++j) {
            int64_t i = g * group + j;
            float t = x[i] * inv;
            t = t + 8.5f;
            int q = (int)t;
            q = q < 0 ? 0 : (q > 15 ? 15 : q);
            if (i & 1) packed[i >> 1] = (uint8_t)((packed[i >> 1] & 0x0f) | (q << 4));
            else packed[i >> 1] = (uint8_t)q;
        }
    }
}

/* GKN twin, _int4_quantize_gkn_kernel int4_gkn_quantize.py:20-75. */
XQO_API void xqo_int4_quantize_gkn(const float* x, uint8_t* packed, float* scales,
                                   int64_t K, int64_t N, int64_t group) {
    const float two_fifteenths = (float)(2.0 / 15.0);
    for (int64_t g = 0; g < K / group; ++g)
        for (int64_t n = 0; n < N; ++n) {
            float amax = 0.0f;
            for (int64_t j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(x[(g * group + j) * N + n]));
            float scale = fmaxf(amax, 1e-12f) * two_fifteenths;
            scales[g * N + n] = scale;
            float inv = 1.0f / scale;
            for (int64_t j = 0; j < group; ++j) {
                int64_t k = g * group + j;
                float t = x[k * N + n] * inv;
                t = t + 8.5f;
                int q = (int)t;
                q = q < 0 ? 0 : (q > 15 ? 15 : q);
                uint8_t* p = &packed[(k >> 1) * N + n];
                if (k & 1) *p = (uint8_t)((*p & 0x0f) | (q << 4));
                else *p = (uint8_t)q;
            }
        }
}

/* The benchmark's symmetric int4 quantizer (not in the reference: it is the
 * rule the workload definition states): scale = bf16(absmax / 7),
 * q = clamp(rne(w / scale), -7, 7) + 8, groups along cols.  Scales are
 * written as bf16 bit patterns. */
XQO_API void xqo_int4_quantize_sym_flat(const float* x, uint8_t* packed, uint16_t* scales_bf16,
                                        int64_t n_elems, int64_t group) {
    for (int64_t g = 0; g < n_elems / group; ++g) {
        float amax = 0.0f;
        for (int64_t j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(x[g * group + j]));
        uint16_t sb = xqo_bf16_rne(amax / 7.0f);
        scales_bf16[g] = sb;
        float scale = xqo_bf16_to_f32(sb);
        for (int64_t j = 0; j < group; ++j) {
            int64_t i = g * group + j;
            int q = 0;
            if (scale > 0.0f) {
                float r = nearbyintf(x[i] / scale);
                r = r < -7.0f ? -7.0f : (r > 7.0f ? 7.0f : r);
                q = (int)r;
            }
            q += 8;
            if (i & 1) packed[i >> 1] = (uint8_t)((packed[i >> 1] & 0x0f) | (q << 4));
            else packed[i >> 1] = (uint8_t)q;
        }
    }
}

/* ------------------------------------------------------------------ */
/* nf4                                                                  */
/* ------------------------------------------------------------------ */

/* The sixteen NormalFloat4 levels, ops/quantize/nf4_codec.py:18-35 (the
 * reference holds them as doubles and builds its fp32 LUT from them, :82-87). */
static const double kNf4Levels[16] = {
    -1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
    -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
    0.07958029955625534, 0.16093020141124725, 0.24611230194568634, 0.33791524171829224,
    0.44070982933044434, 0.5626170039176941, 0.7229568362236023, 1.0};

/* The fifteen decision points of the encoder, nf4_codec.py:48-62. */
static const double kNf4Cuts[15] = {
    -0.8480964004993439, -0.6106329262256622, -0.4599952697753906, -0.3396794348955154,
    -0.2346074059605598, -0.1379117332398891, -0.0455250181257725, 0.0397901497781277,
    0.1202552504837513, 0.2035212516784668, 0.2920137718319893, 0.3893125355243683,
    0.5016634166240692, 0.6427869200706482, 0.8614784181118012};

XQO_API float xqo_nf4_level(int code) { return (float)kNf4Levels[code & 15]; }

/* code = how many decision points lie strictly below v (nf4_codec.py:42-64). */
XQO_API uint8_t xqo_nf4_encode(float v) {
    int code = 0;
    for (int i = 0; i < 15; ++i) code += v > (float)kNf4Cuts[i];
    return (uint8_t)code;
}

/* flat: _nf4_dequantize_kernel, ops/quantize/nf4_quantize.py:62-105: byte i
 * holds element 2i (low nibble) and 2i+1 (high) (:89-90), w =
 * bf16(fl(level[nib] * scale)) with one scale per `group` consecutive elements
 * (:95-103). */
XQO_API void xqo_nf4_decode_flat(const uint8_t* packed, const float* scales,
                                 uint16_t* out, int64_t n_elems, int64_t group) {
    for (int64_t i = 0; i < n_elems; ++i) {
        uint8_t b = packed[i >> 1];
        uint8_t nib = (i & 1) ? (b >> 4) : (b & 0xf);
        float v = (float)kNf4Levels[nib] * scales[i / group];
        out[i] = xqo_bf16_rne(v);
    }
}

/* GKN [K, N]: packed [K/2, N], nibble pairs and groups along K
 * (ops/quantize/nf4_gkn_quantize.py:84-142). */
XQO_API void xqo_nf4_decode_gkn(const uint8_t* packed, const float* scales,
                                uint16_t* out, int64_t K, int64_t N, int64_t group) {
    for (int64_t k = 0; k < K; ++k)
        for (int64_t n = 0; n < N; ++n) {
            uint8_t b = packed[(k >> 1) * N + n];
            uint8_t nib = (k & 1) ? (b >> 4) : (b & 0xf);
            float v = (float)kNf4Levels[nib] * scales[(k / group) * N + n];
            out[k * N + n] = xqo_bf16_rne(v);
        }
}

/* Quantizer, _nf4_quantize_kernel nf4_quantize.py:20-59: scale = max(amax,
 * 1e-12) (:42-43); code = encode(clamp(x * (1/scale), -1, 1)) (:48-52). */
XQO_API void xqo_nf4_quantize_flat(const float* x, uint8_t* packed, float* scales,
                                   int64_t n_elems, int64_t group) {
    for (int64_t g = 0; g < n_elems / group; ++g) {
        float amax = 0.0f;
        for (int64_t j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(x[g * group + j]));
        float scale = fmaxf(amax, 1e-12f);
        scales[g] = scale;
        float inv = 1.0f / scale;
        for (int64_t j = 0; j < group; ++j) {
            int64_t i = g * group + j;
            float t = x[i] * inv;
            t = fminf(fmaxf(t, -1.0f), 1.0f);
            int q = xqo_nf4_encode(t);
            if (i & 1) packed[i >> 1] = (uint8_t)((packed[i >> 1] & 0x0f) | (q << 4));
            else packed[i >> 1] = (uint8_t)q;
        }
    }
}

/* GKN twin, nf4_gkn_quantize.py:22-81. */
XQO_API void xqo_nf4_quantize_gkn(const float* x, uint8_t* packed, float* scales,
                                  int64_t K, int64_t N, int64_t group) {
    for (int64_t g = 0; g < K / group; ++g)
        for (int64_t n = 0; n < N; ++n) {
            float amax = 0.0f;
            for (int64_t j = 0; j < group; ++j) amax = fmaxf(amax, fabsf(x[(g * group + j) * N + n]));
            float scale = fmaxf(amax, 1e-12f);
            scales[g * N + n] = scale;
            float inv = 1.0f / scale;
            for (int64_t j = 0; j < group; ++j) {
                int64_t k = g * group + j;
                float t = x[k * N + n] * inv;
                t = fminf(fmaxf(t, -1.0f), 1.0f);
                int q = xqo_nf4_encode(t);
                uint8_t* p = &packed[(k >> 1) * N + n];
                if (k & 1) *p = (uint8_t)((*p & 0x0f) | (q << 4));
                else *p = (uint8_t)q;
            }
        }
}

/* ------------------------------------------------------------------ */
/* nvfp4                                                                */
/* ------------------------------------------------------------------ */

/* flat: follows _nvfp4_dequantize_kernel, ops/quantize/nvfp4_quantize.py:64-98:
 * sc = fl(float(block_scale) * global) (:81); w = bf16(fl(e2m1(nib) * sc))
 * (:93-96); nibble order as int4.  `scales` is already fp32 here: the caller
 * converts e4m3 bytes with xqo_e4m3_to_f32 (the kernel's .to(f32)). */
XQO_API void xqo_nvfp4_decode_flat(const uint8_t* packed, const float* scales, float global_scale,
                                   uint16_t* out, int64_t n_elems, int64_t block) {
    for (int64_t i = 0; i < n_elems; ++i) {
        uint8_t b = packed[i >> 1];
        uint8_t nib = (i & 1) ? (b >> 4) : (b & 0xf);
        float sc = scales[i / block] * global_scale;
        float v = xqo_e2m1_to_f32(nib) * sc;
        out[i] = xqo_bf16_rne(v);
    }
}

/* GKN: _nvfp4_dequantize_gkn_kernel, ops/quantize/nvfp4_gkn_quantize.py:112-169. */
XQO_API void xqo_nvfp4_decode_gkn(const uint8_t* packed, const float* scales, float global_scale,
                                  uint16_t* out, int64_t K, int64_t N, int64_t block) {
    for (int64_t k = 0; k < K; ++k)
        for (int64_t n = 0; n < N; ++n) {
            uint8_t b = packed[(k >> 1) * N + n];
            uint8_t nib = (k & 1) ? (b >> 4) : (b & 0xf);
            float sc = scales[(k / block) * N + n] * global_scale;
            float v = xqo_e2m1_to_f32(nib) * sc;
            out[k * N + n] = xqo_bf16_rne(v);
        }
}

/* Quantizer, nvfp4_quantize.py:25-60 and :102-111.  Per block amax (>=1e-12);
 * codes from clamp(x * fl(6/amax), +-6) -- encoded against the RAW amax, not
 * the fp8-rounded scale; block_scale = e4m3(fl(fl(amax/gamax) * 448));
 * global = fl(fl(gamax * fl32(1/6)) / 448).  gamax_override < 0 means "use
 * the tensor's own max" (:139-141). Returns global scale. */
static float nvfp4_finish(const float* amax, uint8_t* scales_e4m3, int64_t n_blocks,
                          float gamax_override) {
    float gamax = 0.0f;
    for (int64_t b = 0; b < n_blocks; ++b) gamax = fmaxf(gamax, amax[b]);
    if (gamax_override >= 0.0f) gamax = gamax_override;
    gamax = fmaxf(gamax, 1e-12f);
    for (int64_t b = 0; b < n_blocks; ++b) {
        float t = amax[b] / gamax;
        t = t * 448.0f;
        scales_e4m3[b] = xqo_f32_to_e4m3(t);
    }
    float g = gamax * (float)(1.0 / 6.0);
    return g / 448.0f;
}

XQO_API float xqo_nvfp4_quantize_flat(const float* x, uint8_t* packed, uint8_t* scales_e4m3,
                                      float* amax_buf, int64_t n_elems, int64_t block,
                                      float gamax_override) {
    int64_t nb = n_elems / block;
    for (int64_t b = 0; b < nb; ++b) {
        float amax = 0.0f;
        for (int64_t j = 0; j < block; ++j) amax = fmaxf(amax, fabsf(x[b * block + j]));
        amax = fmaxf(amax, 1e-12f);
        amax_buf[b] = amax;
        float inv = 6.0f / amax;
        for (int64_t j = 0; j < block; ++j) {
            int64_t i = b * block + j;
            float s = x[i] * inv;
            s = fminf(fmaxf(s, -6.0f), 6.0f);
            uint8_t q = xqo_f32_to_e2m1(s);
            if (i & 1) packed[i >> 1] = (uint8_t)((packed[i >> 1] & 0x0f) | (q << 4));
            else packed[i >> 1] = q;
        }
    }
    return nvfp4_finish(amax_buf, scales_e4m3, nb, gamax_override);
}

/* GKN quantizer, nvfp4_gkn_quantize.py:23-108: blocks along K, scales [K/block, N]. */
XQO_API float xqo_nvfp4_quantize_gkn(const float* x, uint8_t* packed, uint8_t* scales_e4m3,
                                     float* amax_buf, int64_t K, int64_t N, int64_t block,
                                     float gamax_override) {
    for (int64_t g = 0; g < K / block; ++g)
        for (int64_t n = 0; n < N; ++n) {
            float amax = 0.0f;
            for (int64_t j = 0; j < block; ++j) amax = fmaxf(amax, fabsf(x[(g * block + j) * N + n]));
            amax = fmaxf(amax, 1e-12f);
            amax_buf[g * N + n] = amax;
            float inv = 6.0f / amax;
            for (int64_t j = 0; j < block; ++j) {
                int64_t k = g * block + j;
                float s = x[k * N + n] * inv;
                s = fminf(fmaxf(s, -6.0f), 6.0f);
                uint8_t q = xqo_f32_to_e2m1(s);
                uint8_t* p = &packed[(k >> 1) * N + n];
                if (k & 1) *p = (uint8_t)((*p & 0x0f) | (q << 4));
                else *p = q;
            }
        }
    return nvfp4_finish(amax_buf, scales_e4m3, (K / block) * N, gamax_override);
}

/* ------------------------------------------------------------------ */
/* block fp8                                                            */
/* ------------------------------------------------------------------ */

/* Follows _block_fp8_dequantize_gkn_kernel, block_fp8_gkn_quantize.py:131-154:
 * p = fl(float(e4m3 byte) * s[i/block][j/block]), stored as fp32 (:171);
 * scale grid is ceil-divided so edge tiles are partial.  The callers' cast
 * (.to(bf16), qlora/modules/linear.py:373) is out_bf16. */
XQO_API void xqo_fp8_decode(const uint8_t* w, const float* scales, float* out_f32,
                            uint16_t* out_bf16, int64_t rows, int64_t cols, int64_t block) {
    int64_t sc = (cols + block - 1) / block;
    for (int64_t i = 0; i < rows; ++i)
        for (int64_t j = 0; j < cols; ++j) {
            float p = xqo_e4m3_to_f32(w[i * cols + j]) * scales[(i / block) * sc + j / block];
            if (out_f32) out_f32[i * cols + j] = p;
            if (out_bf16) out_bf16[i * cols + j] = xqo_bf16_rne(p);
        }
}

/* Follows _block_fp8_quantize_gkn_kernel, block_fp8_gkn_quantize.py:40-70:
 * s = max(fl(fl(amax * amax_scale) / 448), 1e-12); y = e4m3(clamp(fl(x/s), +-448)). */
XQO_API void xqo_fp8_quantize(const float* x, uint8_t* w, float* scales,
                              int64_t rows, int64_t cols, int64_t block, float amax_scale) {
    int64_t sr = (rows + block - 1) / block, sc = (cols + block - 1) / block;
    for (int64_t bi = 0; bi < sr; ++bi)
        for (int64_t bj = 0; bj < sc; ++bj) {
            int64_t i1 = (bi + 1) * block < rows ? (bi + 1) * block : rows;
            int64_t j1 = (bj + 1) * block < cols ? (bj + 1) * block : cols;
            float amax = 0.0f;
            for (int64_t i = bi * block; i < i1; ++i)
                for (int64_t j = bj * block; j < j1; ++j) amax = fmaxf(amax, fabsf(x[i * cols + j]));
            float s = amax * amax_scale;
            s = s / 448.0f;
            s = fmaxf(s, 1e-12f);
            scales[bi * sc + bj] = s;
            for (int64_t i = bi * block; i < i1; ++i)
                for (int64_t j = bj * block; j < j1; ++j) {
                    float y = x[i * cols + j] / s;
                    y = fminf(fmaxf(y, -448.0f), 448.0f);
                    w[i * cols + j] = xqo_f32_to_e4m3(y);
                }
        }
}
