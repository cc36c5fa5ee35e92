// Shared device/host helpers for libxq_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/xq.h"

// ---------------------------------------------------------------- host side
void xq_set_error(const char* fmt, ...);

#define XQ_REQUIRE(cond, ...)            \
    do {                                 \
        if (!(cond)) {                   \
            xq_set_error(__VA_ARGS__);   \
            return XQ_ERR_ARG;           \
        }                                \
    } while (0)

#define XQ_CHECK_LAUNCH(name)                                              \
    do {                                                                   \
        hipError_t e__ = hipGetLastError();                                \
        if (e__ != hipSuccess) {                                           \
            xq_set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
            return XQ_ERR_LAUNCH;                                          \
        }                                                                  \
    } while (0)

int xq_validate_weight(const xq_weight* w, const char* who);
bool xq_profile_mark_begin(hipStream_t s, double flops);
void xq_profile_mark_end(hipStream_t s);
int64_t xq_packed_bytes_per_expert(const xq_weight* w);
int64_t xq_scale_bytes_per_expert(const xq_weight* w);

static inline int64_t xq_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline bool xq_aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

// ---------------------------------------------------------------- vector types
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

typedef uint16_t bf16_t;  // raw bf16 bit pattern in memory

// ---------------------------------------------------------------- scalar codecs
// fp32 -> bf16 bits, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    bf16x2 v;
    v[0] = (__bf16)lo;
    v[1] = (__bf16)hi;
    return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ bf16_t to_bf16(float f) {
    __bf16 b = (__bf16)f;
    return __builtin_bit_cast(bf16_t, b);
}
__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float((uint32_t)h << 16); }

// SwiGLU arithmetic shared by the elementwise kernels and the fused GEMM epilogues (ops/fused_silu_and_mul.py:22-60):
// sigmoid in fp32, the activation rounded to bf16 before it meets `up`
// 1 / (1 + e^-x) with the hardware reciprocal (1 ulp) in place of an IEEE division sequence: the quotient feeds a
// product that is rounded to bf16, and the SwiGLU epilogue of the gate / up launch pays for every instruction here
__device__ __forceinline__ float sigmoid_f32(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float round_bf16(float x) { return bf16_to_f32(to_bf16(x)); }
// The gate pre-activation under a SwiGLU limit (ops/moe/triton.py:127-131, a clamp on the bf16 tensor: the bounds are
// rounded to bf16 with the result); limit <= 0 leaves it alone.  The gate gradient is masked where the unclamped
// value lies outside [-limit, limit] (ops/moe/triton.py:134-141: the bounds themselves are inside).
__device__ __forceinline__ float swiglu_clamp(float g, float limit) {
    return limit > 0.0f ? round_bf16(fminf(fmaxf(g, -limit), limit)) : g;
}
__device__ __forceinline__ float swiglu_mask(float g, float limit) {
    return (limit > 0.0f && !(g >= -limit && g <= limit)) ? 0.0f : 1.0f;
}

// e4m3fn (OCP) byte pair -> two fp32: v_cvt_pk_f32_fp8.  hi selects the upper
// 16 bits of the dword.
__device__ __forceinline__ f32x2 e4m3x2_to_f32(uint32_t word, bool hi) {
    return hi ? __builtin_amdgcn_cvt_pk_f32_fp8(word, true) : __builtin_amdgcn_cvt_pk_f32_fp8(word, false);
}
__device__ __forceinline__ float e4m3_to_f32(uint8_t b) { return __builtin_amdgcn_cvt_pk_f32_fp8((uint32_t)b, false)[0]; }

// e2m1 nibble -> fp32 by bit construction: exponent field c>>1, mantissa bit
// c&1, exponent 0 is the subnormal {0, 0.5}; bit 3 is the sign.
__device__ __forceinline__ float e2m1_to_f32(uint32_t nib) {
    uint32_t c = nib & 7u, e = c >> 1, m = c & 1u;
    uint32_t bits = e ? (((e + 126u) << 23) | (m << 22)) : m * 0x3f000000u;
    return __uint_as_float(bits | ((nib & 8u) << 28));
}

__device__ __forceinline__ float load_scale(const void* p, int64_t idx, int dtype) {
    if (dtype == XQ_SCALE_F32) return ((const float*)p)[idx];
    if (dtype == XQ_SCALE_BF16) return bf16_to_f32(((const bf16_t*)p)[idx]);
    return e4m3_to_f32(((const uint8_t*)p)[idx]);
}

// int4: w = bf16(fl(fl(nib - 8) * s)), as the reference computes it (the
// subtraction is exact; sign of zero follows the multiply).  m8s is unused
// here and kept for the fused form fma(nib, s, -8s), which differs only in
// the sign of a zero result.
__device__ __forceinline__ float int4_val(uint32_t nib, float s, float m8s) {
    (void)m8s;
    return ((float)nib - 8.0f) * s;
}

// NF4 (NormalFloat4) levels, ops/quantize/nf4_codec.py:18-35: w = bf16(fl(level[nib] * scale)).
// A per-lane index into this 64-byte table is a vector load that stays in L1.
static __device__ __constant__ float kNf4Level[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
    0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

// decoded fp32 value of one 4-bit code, before the bf16 rounding; for nvfp4 `s` is already
// fl(block_scale * global_scale)
template <int FMT>
__device__ __forceinline__ float val4(uint32_t nib, float s) {
    if (FMT == XQ_FMT_INT4) return int4_val(nib, s, 0.0f);
    if (FMT == XQ_FMT_NVFP4) return e2m1_to_f32(nib) * s;
    return kNf4Level[nib & 0xfu] * s;
}

// ---------------------------------------------------------------- transposing LDS fragment read
// MFMA 32x32x16 operand fragment from a row-major [k][col] bf16 LDS tile:
__device__ __forceinline__ bf16x8 lds_tr_frag(const bf16_t* tile, int pitch, int krow0, int col0, int lane) {
    // 8 consecutive k (rows krow0 + 8*(lane/32) + 0..7) of column col0 + lane%32,
    // from a row-major [k][col] LDS tile, via two ds_read_b64_tr_b16.
    const int i = lane & 15, g = lane >> 4;
    const bf16_t* base = tile + (krow0 + 8 * (g >> 1) + (i >> 2)) * pitch + col0 + 16 * (g & 1) + 4 * (i & 3);
    typedef __attribute__((ext_vector_type(4))) short s16x4;
    s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(base));
    s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4 __attribute__((address_space(3)))*)(base + 4 * pitch));
    typedef __attribute__((ext_vector_type(8))) short s16x8;
    s16x8 v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    return __builtin_bit_cast(bf16x8, v);
}

