// Shared by the two organisations of the skinny-M forward (xq_skinny.hip: K split over blocks, two launches;
// xq_skinny_rows.hip: whole rows per block, one launch).
#pragma once
#include "xq_common.h"

namespace xq {

// decode 8 consecutive K elements (one MFMA operand) of this lane's row
template <int FMT>
__device__ __forceinline__ bf16x8 decode8(uint32_t w0, uint32_t w1, float s0, float s1, const float* nf4_lds = nullptr) {
    uint32_t o[4];
    if (FMT == XQ_FMT_FP8) {
        f32x2 a = e4m3x2_to_f32(w0, false), b = e4m3x2_to_f32(w0, true);
        f32x2 c = e4m3x2_to_f32(w1, false), d = e4m3x2_to_f32(w1, true);
        o[0] = pack_bf16x2(a[0] * s0, a[1] * s0);
        o[1] = pack_bf16x2(b[0] * s0, b[1] * s0);
        o[2] = pack_bf16x2(c[0] * s0, c[1] * s0);
        o[3] = pack_bf16x2(d[0] * s0, d[1] * s0);
    } else if (FMT == XQ_FMT_INT4) {
        // w0 holds 8 nibbles; fma(nib, s, -8s) == fl((nib-8)*s) up to the sign of zero.  The nibbles become floats two
        // at a time through the fp8 converter: a byte 0x0n read as e4m3 is n * 2^-9 for every n in 0..15 (the subnormals
        // run without a gap into the first binade), and (n * 2^-9) * (512 s) is n * s exactly.
        const uint32_t ev = w0 & 0x0f0f0f0fu, od = (w0 >> 4) & 0x0f0f0f0fu;     // nibbles 0 2 4 6 / 1 3 5 7, one per byte
        const float s512 = s0 * 512.0f;
        const f32x2 e01 = e4m3x2_to_f32(ev, false), e23 = e4m3x2_to_f32(ev, true);
        const f32x2 o01 = e4m3x2_to_f32(od, false), o23 = e4m3x2_to_f32(od, true);
        o[0] = pack_bf16x2(__builtin_fmaf(e01[0], s512, s1), __builtin_fmaf(o01[0], s512, s1));
        o[1] = pack_bf16x2(__builtin_fmaf(e01[1], s512, s1), __builtin_fmaf(o01[1], s512, s1));
        o[2] = pack_bf16x2(__builtin_fmaf(e23[0], s512, s1), __builtin_fmaf(o23[0], s512, s1));
        o[3] = pack_bf16x2(__builtin_fmaf(e23[1], s512, s1), __builtin_fmaf(o23[1], s512, s1));
    } else if (FMT == XQ_FMT_NF4) {
        // level[nib] * scale, the levels read from a 64-byte copy of the table in LDS (conflict free for any mix of codes)
#pragma unroll
        for (int i = 0; i < 4; ++i)
            o[i] = pack_bf16x2(nf4_lds[(w0 >> (8 * i)) & 0xfu] * s0, nf4_lds[(w0 >> (8 * i + 4)) & 0xfu] * s0);
    } else {
        // v_cvt_scalef32_pk_f32_fp4 with scale 1.0 yields the exact e2m1 values of byte i (low nibble first)
        f32x2 v0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w0, 1.0f, 0);
        f32x2 v1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w0, 1.0f, 1);
        f32x2 v2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w0, 1.0f, 2);
        f32x2 v3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w0, 1.0f, 3);
        o[0] = pack_bf16x2(v0[0] * s0, v0[1] * s0);
        o[1] = pack_bf16x2(v1[0] * s0, v1[1] * s0);
        o[2] = pack_bf16x2(v2[0] * s0, v2[1] * s0);
        o[3] = pack_bf16x2(v3[0] * s0, v3[1] * s0);
    }
    u32x4 r = {o[0], o[1], o[2], o[3]};
    return __builtin_bit_cast(bf16x8, r);
}

void set_skinny_rows(int enabled);
bool skinny_rows_enabled();
void set_skinny_rows_spin_limit(int limit);   // <= 0: the default
void set_skinny_gemv(int on);                  // M = 1 on the dot-product kernel (default) or on the MFMA kernel
bool skinny_gemv_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r);
int launch_skinny_gemv(const xq_weight* w, const bf16_t* x, const void* lora_A, const void* lora_B, int r, float scaling,
                       const bf16_t* bias, bf16_t* y, const void* slot_key, hipStream_t stream, bool swiglu);
int reset_skinny_rows_slots();                 // clears the current device's slots (synchronises the device)
int skinny_rows_status(int* gave_up, int* failed_slots, hipStream_t stream);   // reads and clears the failure reports (synchronises the stream)

// ---- one-launch organisation (xq_skinny_rows.hip)
// true when the shape, format and LoRA operands fit it; the caller falls back to the split organisation otherwise
bool skinny_rows_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r);
// `slot_key` names the caller's scratch (its workspace pointer): calls with different keys may overlap on a device
int launch_skinny_rows(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B, int r,
                       float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, const void* slot_key, hipStream_t stream);

// gate | up as one weight [2 I, K] with the SwiGLU finish: h [M, I] = silu(gate) * up in one launch
bool skinny_rows_swiglu_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r);
int launch_skinny_rows_swiglu(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B, int r,
                              float scaling, const bf16_t* bias, bf16_t* h, int64_t ldh, const void* slot_key, hipStream_t stream);

// several forwards that share x (same format, K and M) as one launch of the same kernel; each forward has its own slot,
// keyed by addresses 256 bytes apart from `slot_key` (the caller's workspace holds at least 256 bytes per forward)
struct SkinnyRowsJob {
    const xq_weight* w;
    const void* lora_A;
    const void* lora_B;
    int r;
    float scaling;
    const bf16_t* bias;
    bf16_t* y;
    int64_t ldy;
};
bool skinny_rows_multi_supported(const SkinnyRowsJob* jobs, int n_jobs, int64_t M, int lora_dtype);
int launch_skinny_rows_multi(const SkinnyRowsJob* jobs, int n_jobs, const bf16_t* x, int64_t ldx, int64_t M, const void* slot_key,
                             hipStream_t stream);

}  // namespace xq
