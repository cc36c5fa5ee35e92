// Merging the LoRA update into the quantized base weight without materialising it:
//
//   W'[n, k] = deq(W)[n, k] + scaling * sum_j B[n, j] * A[j, k]          (W FLAT [N, K])
//
// One block owns a 128 x 128 tile -- exactly one block-fp8 scale block -- and
//   1. computes the tile of the low-rank product on the matrix cores.  The reference
//      multiplies the fp32 factors in fp32; here each factor is split into two bf16
//      terms (hi + lo, 16 significant bits) and the product is the three bf16 MFMA
//      products hi*hi + hi*lo + lo*hi with fp32 accumulation (relative error ~2^-16
//      per term instead of 2^-9 with plain bf16 factors);
//   2. parks it in LDS, then walks the tile row-contiguously: every thread owns 64
//      consecutive columns of one row, loads the packed codes with 16-byte loads,
//      decodes them to the reference decoder's value and adds the update;
//   3a. (publish) rounds to bf16 -- bf16(bf16(deq) + bf16(delta)), the arithmetic of the
//      reference's weight-sync merge -- or writes the fp32 sum; or
//   3b. (requantise, block-fp8) reduces the tile's absmax, derives the new block scale
//      s = max(amax / 448, 1e-12) and writes e4m3(clamp(x / s)) bytes and the scale:
//      decode -> add -> re-encode in one pass over 1 byte per weight each way.
#include "xq_common.h"
#include "xq_lora.h"

namespace xq {

constexpr int MG_T = 128;           // tile edge
constexpr int MG_FP = 64 + 8;       // factor tile row pitch (bf16 elements): 144 B
constexpr int MG_DP = MG_T + 4;     // delta tile row pitch (floats)

struct MergeArgs {
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int32_t fmt, group, scale_dtype;
    int32_t N, K;
    const void* A;       // [r, K]
    const void* B;       // [N, r]
    int32_t lora_f32, r, r_pad;
    float scaling;
    int32_t mode;        // 0: bf16 out (publish arithmetic), 1: fp32 out, 2: block-fp8 requantise
    void* out;           // mode 0/1: [N, K]
    uint8_t* packed_out; // mode 2: [N, K] e4m3 bytes    } both may alias the inputs: a block reads its tile and its
    float* scales_out;   // mode 2: [ceil(N/128), ceil(K/128)] } scale before it writes them, and touches no other
};

__device__ __forceinline__ float factor_at(const void* p, int64_t idx, bool f32) {
    return f32 ? ((const float*)p)[idx] : bf16_to_f32(((const bf16_t*)p)[idx]);
}

// decode 16 consecutive elements of row n starting at column k (k % 16 == 0) to fp32, exactly as xq_decode does
template <int FMT>
__device__ __forceinline__ void decode_run16(const MergeArgs& g, int64_t n, int k, float* v) {
    if (FMT == XQ_FMT_FP8) {
        const u32x4 w = *(const u32x4*)(g.packed + n * g.K + k);
        const float s = ((const float*)g.scales)[(n >> 7) * ((g.K + 127) >> 7) + (k >> 7)];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const f32x2 lo = e4m3x2_to_f32(w[i], false), hi = e4m3x2_to_f32(w[i], true);
            v[4 * i] = lo[0] * s; v[4 * i + 1] = lo[1] * s; v[4 * i + 2] = hi[0] * s; v[4 * i + 3] = hi[1] * s;
        }
    } else {
        const u32x2 w = *(const u32x2*)(g.packed + ((n * g.K + k) >> 1));
        const float gs = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const uint32_t nib = (w[i >> 3] >> (4 * (i & 7))) & 0xfu;
            // one scale per `group` elements; group is even, so a pair never straddles two groups
            const float s = load_scale(g.scales, (n * g.K + k + i) / g.group, g.scale_dtype);
            v[i] = val4<FMT>(nib, FMT == XQ_FMT_NVFP4 ? s * gs : s);
        }
    }
}

template <int FMT, int RP>
__global__ void __launch_bounds__(256) merge_kernel(MergeArgs g) {
    extern __shared__ __attribute__((aligned(16))) uint8_t mg_lds[];
    __shared__ float sh_amax[4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int k0 = blockIdx.x * MG_T, n0 = blockIdx.y * MG_T;
    constexpr int rp = RP;        // LoRA rank rounded up to 16 (0: no update)
    float* dt = (float*)mg_lds;   // delta tile [128][MG_DP] (used after the factor tiles are dead)

    if (rp > 0) {
        // ---- 1. factor tiles, split hi/lo, both [row][j]: Bt rows = n, At rows = k
        bf16_t* Bh = (bf16_t*)mg_lds;
        bf16_t* Bl = Bh + MG_T * MG_FP;
        bf16_t* Ah = Bl + MG_T * MG_FP;
        bf16_t* Al = Ah + MG_T * MG_FP;
        const bool f32 = g.lora_f32 != 0;
        // every load of a factor tile is issued before its first use (compile-time trip counts)
        {
            constexpr int H = RP / 2;                     // thread -> row tid >> 1, ranks (tid & 1) * H .. +H
            const int row = tid >> 1, j0 = (tid & 1) * H;
            const int64_t n = n0 + row;
            float v[H > 0 ? H : 1];
#pragma unroll
            for (int jj = 0; jj < H; ++jj) v[jj] = (j0 + jj < g.r && n < g.N) ? factor_at(g.B, n * g.r + j0 + jj, f32) : 0.0f;
#pragma unroll
            for (int jj = 0; jj < H; jj += 2) {
                const bf16_t h0 = to_bf16(v[jj]), h1 = to_bf16(v[jj + 1]);
                *(uint32_t*)(Bh + row * MG_FP + j0 + jj) = (uint32_t)h0 | ((uint32_t)h1 << 16);
                *(uint32_t*)(Bl + row * MG_FP + j0 + jj) = pack_bf16x2(v[jj] - bf16_to_f32(h0), v[jj + 1] - bf16_to_f32(h1));
            }
        }
        {
            constexpr int H = RP / 2;                     // thread -> column tid & 127, ranks (tid >> 7) * H .. +H
            const int kk = tid & 127, j0 = (tid >> 7) * H;   // consecutive threads along k: coalesced rows of A
            const int64_t k = k0 + kk;
            float v[H > 0 ? H : 1];
#pragma unroll
            for (int jj = 0; jj < H; ++jj) v[jj] = (j0 + jj < g.r && k < g.K) ? factor_at(g.A, (int64_t)(j0 + jj) * g.K + k, f32) : 0.0f;
#pragma unroll
            for (int jj = 0; jj < H; jj += 2) {
                const bf16_t h0 = to_bf16(v[jj]), h1 = to_bf16(v[jj + 1]);
                *(uint32_t*)(Ah + kk * MG_FP + j0 + jj) = (uint32_t)h0 | ((uint32_t)h1 << 16);
                *(uint32_t*)(Al + kk * MG_FP + j0 + jj) = pack_bf16x2(v[jj] - bf16_to_f32(h0), v[jj + 1] - bf16_to_f32(h1));
            }
        }
        __syncthreads();
        // ---- 2. delta tile on the matrix cores: wave (wm, wn) owns rows wm*64.., cols wn*64..
        const int wm = wave >> 1, wn = wave & 1, fr = lane & 31, fk = (lane >> 5) * 8;
        f32x16 acc[2][2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;
        for (int ks = 0; ks < (rp >> 4); ++ks) {
            bf16x8 bh[2], bl[2], ah[2], al[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int ro = (wm * 64 + i * 32 + fr) * MG_FP + ks * 16 + fk;
                const int co = (wn * 64 + i * 32 + fr) * MG_FP + ks * 16 + fk;
                bh[i] = *(const bf16x8*)(Bh + ro); bl[i] = *(const bf16x8*)(Bl + ro);
                ah[i] = *(const bf16x8*)(Ah + co); al[i] = *(const bf16x8*)(Al + co);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bl[i], ah[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh[i], al[j], acc[i][j], 0, 0, 0);
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh[i], ah[j], acc[i][j], 0, 0, 0);
                }
        }
        __syncthreads();   // factor tiles are dead: the delta tile takes their place
        const int rgrp = (lane >> 5) * 4;
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const int row = wm * 64 + i * 32 + (q & 3) + rgrp + 8 * (q >> 2), col = wn * 64 + j * 32 + fr;
                    dt[row * MG_DP + col] = acc[i][j][q] * g.scaling;
                }
        __syncthreads();
    }

    // ---- 3. row-contiguous pass: thread -> row tid >> 1, columns (tid & 1) * 64 .. +64
    const int row = tid >> 1, c0 = (tid & 1) * 64;
    const int64_t n = n0 + row;
    const bool row_ok = n < g.N;
    float m[64];
    float amax = 0.0f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int k = k0 + c0 + u * 16;
        const bool ok = row_ok && k < g.K;   // K % 16 == 0: runs are all in or all out
        float v[16];
        if (ok) decode_run16<FMT>(g, n, k, v);
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const float d = rp > 0 ? dt[row * MG_DP + c0 + u * 16 + i] : 0.0f;
            float x;
            if (g.mode == 0) x = bf16_to_f32(to_bf16(bf16_to_f32(to_bf16(v[i])) + bf16_to_f32(to_bf16(d))));
            else if (FMT == XQ_FMT_FP8) x = v[i] + d;
            else x = bf16_to_f32(to_bf16(bf16_to_f32(to_bf16(v[i])) + bf16_to_f32(to_bf16(d))));   // 4-bit decoders return bf16
            x = ok ? x : 0.0f;
            m[u * 16 + i] = x;
            amax = fmaxf(amax, fabsf(x));
        }
    }
    if (g.mode != 2) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int k = k0 + c0 + u * 16;
            if (!(row_ok && k < g.K)) continue;
            if (g.mode == 0) {
                bf16_t* o = (bf16_t*)g.out + n * g.K + k;
                uint32_t pk[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) pk[i] = pack_bf16x2(m[u * 16 + 2 * i], m[u * 16 + 2 * i + 1]);
                *(u32x4*)o = u32x4{pk[0], pk[1], pk[2], pk[3]};
                *(u32x4*)(o + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
            } else {
                float* o = (float*)g.out + n * g.K + k;
#pragma unroll
                for (int i = 0; i < 4; ++i) *(f32x4*)(o + 4 * i) = f32x4{m[u * 16 + 4 * i], m[u * 16 + 4 * i + 1], m[u * 16 + 4 * i + 2], m[u * 16 + 4 * i + 3]};
            }
        }
        return;
    }
    // ---- 3b. block absmax -> new scale -> e4m3 bytes
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) sh_amax[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(sh_amax[0], sh_amax[1]), fmaxf(sh_amax[2], sh_amax[3]));
    const float s = fmaxf(amax / 448.0f, 1e-12f);
    if (tid == 0) g.scales_out[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = s;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int k = k0 + c0 + u * 16;
        if (!(row_ok && k < g.K)) continue;
        uint32_t pk[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = fminf(fmaxf(m[u * 16 + 4 * i + e] / s, -448.0f), 448.0f);
            uint32_t w = 0;
            w = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w, false);
            w = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w, true);
            pk[i] = w;
        }
        *(u32x4*)(g.packed_out + n * g.K + k) = u32x4{pk[0], pk[1], pk[2], pk[3]};
    }
}

}  // namespace xq

using namespace xq;

// FLOP-free roofline figure of this path: bytes in + bytes out per launch
static double merge_bytes(const xq_weight* w, int mode) {
    const double n = (double)w->rows * w->cols;
    const double in = (double)xq_packed_bytes_per_expert(w) + (double)xq_scale_bytes_per_expert(w);
    return in + (mode == 0 ? 2.0 * n : mode == 1 ? 4.0 * n : in);
}

template <int FMT, int RP>
static int launch_merge_one(const MergeArgs& g, dim3 grid, size_t lds, hipStream_t s, const char* who) {
    static bool attr_set = false;   // per instantiation
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)merge_kernel<FMT, RP>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            xq_set_error("%s: cannot raise the dynamic LDS limit: %s", who, hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    merge_kernel<FMT, RP><<<grid, 256, lds, s>>>(g);
    return XQ_OK;
}

template <int FMT>
static int launch_merge_fmt(const MergeArgs& g, dim3 grid, size_t lds, hipStream_t s, const char* who) {
    switch (g.r_pad) {
        case 0: return launch_merge_one<FMT, 0>(g, grid, lds, s, who);
        case 16: return launch_merge_one<FMT, 16>(g, grid, lds, s, who);
        case 32: return launch_merge_one<FMT, 32>(g, grid, lds, s, who);
        case 48: return launch_merge_one<FMT, 48>(g, grid, lds, s, who);
        default: return launch_merge_one<FMT, 64>(g, grid, lds, s, who);
    }
}

static int launch_merge(const xq_weight* w, const void* A, const void* B, int lora_dtype, int r, float scaling, int mode,
                        void* out, void* packed_out, float* scales_out, hipStream_t stream, const char* who) {
    int rc = xq_validate_weight(w, who);
    if (rc) return rc;
    XQ_REQUIRE(w->num_experts == 1, "%s: takes a single matrix", who);
    XQ_REQUIRE(w->format == XQ_FMT_FP8 || w->layout == XQ_LAYOUT_FLAT, "%s: dense weights are FLAT [N, K]", who);
    XQ_REQUIRE(w->cols % 16 == 0, "%s: in_features %lld must be a multiple of 16", who, (long long)w->cols);
    XQ_REQUIRE(r >= 0 && r <= 64, "%s: LoRA rank %d out of range [0, 64]", who, r);
    XQ_REQUIRE(r == 0 || (A && B), "%s: LoRA factors are NULL", who);
    XQ_REQUIRE(lora_dtype == XQ_DT_F32 || lora_dtype == XQ_DT_BF16, "%s: bad lora_dtype", who);
    XQ_REQUIRE(xq_aligned(w->packed, 16), "%s: packed weight must be 16-byte aligned", who);
    if (w->rows == 0 || w->cols == 0) return XQ_OK;
    MergeArgs g;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.fmt = w->format; g.group = w->group; g.scale_dtype = w->scale_dtype;
    g.N = (int32_t)w->rows; g.K = (int32_t)w->cols;
    g.A = A; g.B = B; g.lora_f32 = lora_dtype == XQ_DT_F32; g.r = r; g.r_pad = r <= 0 ? 0 : ((r + 15) / 16) * 16;
    g.scaling = scaling; g.mode = mode; g.out = out; g.packed_out = (uint8_t*)packed_out; g.scales_out = scales_out;
    const size_t lds_f = (size_t)4 * MG_T * MG_FP * 2, lds_d = (size_t)MG_T * MG_DP * 4;
    const size_t lds = lds_f > lds_d ? lds_f : lds_d;
    dim3 grid((unsigned)xq_cdiv(w->cols, MG_T), (unsigned)xq_cdiv(w->rows, MG_T));
    const bool timed = xq_profile_mark_begin(stream, merge_bytes(w, mode));
    if (w->format == XQ_FMT_FP8) rc = launch_merge_fmt<XQ_FMT_FP8>(g, grid, lds, stream, who);
    else if (w->format == XQ_FMT_INT4) rc = launch_merge_fmt<XQ_FMT_INT4>(g, grid, lds, stream, who);
    else if (w->format == XQ_FMT_NF4) rc = launch_merge_fmt<XQ_FMT_NF4>(g, grid, lds, stream, who);
    else rc = launch_merge_fmt<XQ_FMT_NVFP4>(g, grid, lds, stream, who);
    if (timed) xq_profile_mark_end(stream);
    if (rc) return rc;
    XQ_CHECK_LAUNCH(who);
    return XQ_OK;
}

extern "C" int xq_merge_dense(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                              float scaling, void* out, int out_dtype, void* stream) {
    XQ_REQUIRE(out_dtype == XQ_DT_BF16 || out_dtype == XQ_DT_F32, "xq_merge_dense: bad out_dtype");
    XQ_REQUIRE(out && xq_aligned(out, 16), "xq_merge_dense: out is NULL or not 16-byte aligned");
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, out_dtype == XQ_DT_BF16 ? 0 : 1, out, nullptr, nullptr,
                        (hipStream_t)stream, "xq_merge_dense");
}

extern "C" int xq_merge_requant_fp8(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                                    float scaling, void* packed_out, float* scales_out, void* stream) {
    XQ_REQUIRE(w && w->format == XQ_FMT_FP8, "xq_merge_requant_fp8: the weight must be block_fp8");
    XQ_REQUIRE(packed_out && scales_out && xq_aligned(packed_out, 16), "xq_merge_requant_fp8: NULL or misaligned output");
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, 2, nullptr, packed_out, scales_out, (hipStream_t)stream,
                        "xq_merge_requant_fp8");
}
