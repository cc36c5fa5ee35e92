// Stand-alone weight decode: packed int4 / nvfp4 / nf4 / block-fp8 -> bf16 (or fp32).
// HBM-bound: every thread moves 16 B of packed codes and writes the decoded
// run with 16 B stores.  Bit-exact with the reference decoders:
//   int4   (nib-8)*scale                    ops/quantize/int4_quantize.py:45-76, int4_gkn_quantize.py:79-130
//   nvfp4  e2m1(nib)*(block_scale*global)   ops/quantize/nvfp4_quantize.py:64-98, nvfp4_gkn_quantize.py:112-169
//   nf4    level[nib]*scale                 ops/quantize/nf4_quantize.py:61-105, nf4_gkn_quantize.py:84-138
//   fp8    float(e4m3)*s[i/128][j/128]      ops/quantize/block_fp8_gkn_quantize.py:131-154
#include "xq_common.h"

namespace {

struct DecodeArgs {
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    void* out;
    int64_t rows, cols;
    int64_t packed_stride, scale_stride;  // bytes per expert
    int32_t group, scale_dtype;
};

template <bool F32>
__device__ __forceinline__ void store_run16(void* out, int64_t idx, const float* v) {
    if (F32) {
        f32x4* o = (f32x4*)((float*)out + idx);
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = f32x4{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
    } else {
        u32x4* o = (u32x4*)((bf16_t*)out + idx);
#pragma unroll
        for (int i = 0; i < 2; ++i)
            o[i] = u32x4{pack_bf16x2(v[8 * i], v[8 * i + 1]), pack_bf16x2(v[8 * i + 2], v[8 * i + 3]),
                         pack_bf16x2(v[8 * i + 4], v[8 * i + 5]), pack_bf16x2(v[8 * i + 6], v[8 * i + 7])};
    }
}

// ------------------------------------------------------------------ fp8
// one thread = 16 consecutive bytes of one row (cols % 16 == 0)
template <bool F32>
__global__ void __launch_bounds__(256) decode_fp8_vec(DecodeArgs a, int64_t chunks_per_row, int64_t total) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int64_t per_expert = a.rows * chunks_per_row;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    int64_t row = rem / chunks_per_row, c0 = (rem - row * chunks_per_row) * 16;
    const uint8_t* p = a.packed + e * a.packed_stride + row * a.cols + c0;
    u32x4 w = *(const u32x4*)p;
    int64_t sc = (a.cols + 127) / 128;
    const float* sp = (const float*)(a.scales + e * a.scale_stride);
    float s = sp[(row >> 7) * sc + (c0 >> 7)];
    float v[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f32x2 lo = e4m3x2_to_f32(w[i], false), hi = e4m3x2_to_f32(w[i], true);
        v[4 * i] = lo[0] * s;
        v[4 * i + 1] = lo[1] * s;
        v[4 * i + 2] = hi[0] * s;
        v[4 * i + 3] = hi[1] * s;
    }
    store_run16<F32>(a.out, (e * a.rows + row) * a.cols + c0, v);
}

template <bool F32>
__global__ void __launch_bounds__(256) decode_fp8_scalar(DecodeArgs a, int64_t total) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int64_t per_expert = a.rows * a.cols;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    int64_t row = rem / a.cols, col = rem - row * a.cols;
    int64_t sc = (a.cols + 127) / 128;
    float s = ((const float*)(a.scales + e * a.scale_stride))[(row >> 7) * sc + (col >> 7)];
    float v = e4m3_to_f32(a.packed[e * a.packed_stride + rem]) * s;
    if (F32) ((float*)a.out)[t] = v;
    else ((bf16_t*)a.out)[t] = to_bf16(v);
}

// ------------------------------------------------------------------ 4-bit, FLAT
// one thread = 8 packed bytes = 16 consecutive elements of a row
// (cols % 16 == 0 and group % 16 == 0: the run lies in one scale group)
template <int FMT>
__global__ void __launch_bounds__(256) decode_4bit_flat_vec(DecodeArgs a, int64_t chunks_per_row, int64_t total) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int64_t per_expert = a.rows * chunks_per_row;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    int64_t row = rem / chunks_per_row, c0 = (rem - row * chunks_per_row) * 16;
    u32x2 w = *(const u32x2*)(a.packed + e * a.packed_stride + (row * a.cols + c0) / 2);
    int64_t gidx = (row * a.cols + c0) / a.group;
    float s = load_scale(a.scales + e * a.scale_stride, gidx, a.scale_dtype);
    float v[16];
    if (FMT == XQ_FMT_NVFP4) s = s * a.global_scale[e];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = val4<FMT>((w[i >> 3] >> (4 * (i & 7))) & 0xfu, s);
    store_run16<false>(a.out, (e * a.rows + row) * a.cols + c0, v);
}

// one thread = one packed byte = 2 consecutive elements (any even cols/group)
template <int FMT>
__global__ void __launch_bounds__(256) decode_4bit_flat_scalar(DecodeArgs a, int64_t total_bytes) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total_bytes) return;
    int64_t per_expert = a.rows * a.cols / 2;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    uint32_t b = a.packed[e * a.packed_stride + rem];
    float s = load_scale(a.scales + e * a.scale_stride, (rem * 2) / a.group, a.scale_dtype);
    if (FMT == XQ_FMT_NVFP4) s = s * a.global_scale[e];
    const float lo = val4<FMT>(b & 0xfu, s), hi = val4<FMT>(b >> 4, s);
    ((uint32_t*)a.out)[t] = pack_bf16x2(lo, hi);
}

// ------------------------------------------------------------------ 4-bit, GKN
// packed [rows/2, cols]; one thread = 16 bytes of a packed row = rows (2r, 2r+1) x 16 cols
template <int FMT>
__global__ void __launch_bounds__(256) decode_4bit_gkn_vec(DecodeArgs a, int64_t chunks_per_row, int64_t total) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int64_t per_expert = (a.rows / 2) * chunks_per_row;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    int64_t r2 = rem / chunks_per_row, c0 = (rem - r2 * chunks_per_row) * 16;
    u32x4 w = *(const u32x4*)(a.packed + e * a.packed_stride + r2 * a.cols + c0);
    int64_t g = (2 * r2) / a.group;
    const uint8_t* sp = a.scales + e * a.scale_stride;
    float gs = FMT == XQ_FMT_NVFP4 ? a.global_scale[e] : 1.0f;
    float ve[16], vo[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        uint32_t b = (w[i >> 2] >> (8 * (i & 3))) & 0xffu;
        float s = load_scale(sp, g * a.cols + c0 + i, a.scale_dtype);
        if (FMT == XQ_FMT_NVFP4) s = s * gs;
        ve[i] = val4<FMT>(b & 0xfu, s);
        vo[i] = val4<FMT>(b >> 4, s);
    }
    int64_t base = (e * a.rows + 2 * r2) * a.cols + c0;
    store_run16<false>(a.out, base, ve);
    store_run16<false>(a.out, base + a.cols, vo);
}

template <int FMT>
__global__ void __launch_bounds__(256) decode_4bit_gkn_scalar(DecodeArgs a, int64_t total_bytes) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total_bytes) return;
    int64_t per_expert = (a.rows / 2) * a.cols;
    int64_t e = t / per_expert, rem = t - e * per_expert;
    int64_t r2 = rem / a.cols, c = rem - r2 * a.cols;
    uint32_t b = a.packed[e * a.packed_stride + rem];
    float s = load_scale(a.scales + e * a.scale_stride, ((2 * r2) / a.group) * a.cols + c, a.scale_dtype);
    if (FMT == XQ_FMT_NVFP4) s = s * a.global_scale[e];
    const float lo = val4<FMT>(b & 0xfu, s), hi = val4<FMT>(b >> 4, s);
    bf16_t* o = (bf16_t*)a.out + (e * a.rows + 2 * r2) * a.cols + c;
    o[0] = to_bf16(lo);
    o[a.cols] = to_bf16(hi);
}

inline dim3 grid_for(int64_t n) { return dim3((unsigned)xq_cdiv(n, 256)); }

}  // namespace

extern "C" int xq_decode(const xq_weight* w, void* out, int out_dtype, void* stream_) {
    int rc = xq_validate_weight(w, "xq_decode");
    if (rc) return rc;
    XQ_REQUIRE(out != nullptr || w->rows == 0 || w->cols == 0, "xq_decode: out is NULL");
    XQ_REQUIRE(out_dtype == XQ_DT_BF16 || out_dtype == XQ_DT_F32, "xq_decode: bad out_dtype %d", out_dtype);
    XQ_REQUIRE(out_dtype == XQ_DT_BF16 || w->format == XQ_FMT_FP8,
               "xq_decode: fp32 output is only defined for block_fp8 (the 4-bit reference decoders emit bf16)");
    hipStream_t stream = (hipStream_t)stream_;
    DecodeArgs a;
    a.packed = (const uint8_t*)w->packed;
    a.scales = (const uint8_t*)w->scales;
    a.global_scale = w->global_scale;
    a.out = out;
    a.rows = w->rows;
    a.cols = w->cols;
    a.packed_stride = xq_packed_bytes_per_expert(w);
    a.scale_stride = xq_scale_bytes_per_expert(w);
    a.group = w->group;
    a.scale_dtype = w->scale_dtype;
    int64_t E = w->num_experts;
    if (w->rows == 0 || w->cols == 0) return XQ_OK;
    int64_t elems = E * w->rows * w->cols;
    XQ_REQUIRE(elems / 2 < ((int64_t)1 << 39), "xq_decode: tensor too large");

    if (w->format == XQ_FMT_FP8) {
        bool vec = (w->cols % 16 == 0) && xq_aligned(w->packed, 16) && xq_aligned(out, 16) && (a.packed_stride % 16 == 0);
        if (vec) {
            int64_t cpr = w->cols / 16, total = E * w->rows * cpr;
            if (out_dtype == XQ_DT_F32) decode_fp8_vec<true><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
            else decode_fp8_vec<false><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
        } else {
            if (out_dtype == XQ_DT_F32) decode_fp8_scalar<true><<<grid_for(elems), 256, 0, stream>>>(a, elems);
            else decode_fp8_scalar<false><<<grid_for(elems), 256, 0, stream>>>(a, elems);
        }
    } else if (w->layout == XQ_LAYOUT_FLAT) {
        bool vec = (w->cols % 16 == 0) && (w->group % 16 == 0) && xq_aligned(w->packed, 8) && xq_aligned(out, 16) &&
                   (a.packed_stride % 8 == 0);
        if (vec) {
            int64_t cpr = w->cols / 16, total = E * w->rows * cpr;
            if (w->format == XQ_FMT_INT4) decode_4bit_flat_vec<XQ_FMT_INT4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
            else if (w->format == XQ_FMT_NVFP4) decode_4bit_flat_vec<XQ_FMT_NVFP4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
            else decode_4bit_flat_vec<XQ_FMT_NF4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
        } else {
            int64_t total = elems / 2;
            XQ_REQUIRE(xq_aligned(out, 4), "xq_decode: out must be 4-byte aligned");
            if (w->format == XQ_FMT_INT4) decode_4bit_flat_scalar<XQ_FMT_INT4><<<grid_for(total), 256, 0, stream>>>(a, total);
            else if (w->format == XQ_FMT_NVFP4) decode_4bit_flat_scalar<XQ_FMT_NVFP4><<<grid_for(total), 256, 0, stream>>>(a, total);
            else decode_4bit_flat_scalar<XQ_FMT_NF4><<<grid_for(total), 256, 0, stream>>>(a, total);
        }
    } else {
        bool vec = (w->cols % 16 == 0) && xq_aligned(w->packed, 16) && xq_aligned(out, 16) && (a.packed_stride % 16 == 0);
        if (vec) {
            int64_t cpr = w->cols / 16, total = E * (w->rows / 2) * cpr;
            if (w->format == XQ_FMT_INT4) decode_4bit_gkn_vec<XQ_FMT_INT4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
            else if (w->format == XQ_FMT_NVFP4) decode_4bit_gkn_vec<XQ_FMT_NVFP4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
            else decode_4bit_gkn_vec<XQ_FMT_NF4><<<grid_for(total), 256, 0, stream>>>(a, cpr, total);
        } else {
            int64_t total = elems / 2;
            if (w->format == XQ_FMT_INT4) decode_4bit_gkn_scalar<XQ_FMT_INT4><<<grid_for(total), 256, 0, stream>>>(a, total);
            else if (w->format == XQ_FMT_NVFP4) decode_4bit_gkn_scalar<XQ_FMT_NVFP4><<<grid_for(total), 256, 0, stream>>>(a, total);
            else decode_4bit_gkn_scalar<XQ_FMT_NF4><<<grid_for(total), 256, 0, stream>>>(a, total);
        }
    }
    XQ_CHECK_LAUNCH("xq_decode");
    return XQ_OK;
}
