// Skinny-M (M <= 64) fused dequant-GEMM forward: the HBM-bound decode/rollout regime.
//
//   y[M, N] = x[M, K] . deq(W)^T + bias + su[M, r] . Lr[N, r]^T          (W FLAT [N, K])
//
// The packed weight is streamed from HBM exactly once, straight into the MFMA
// operand registers: lane (n, h) of a wave owns row n of a 32-row slab and the
// h-th 64-element half of each 128-element K chunk, so the four 16-byte loads a
// lane issues per chunk (two for 4-bit formats) cover whole 128-byte lines and
// every line is used once.  The bytes are decoded in registers to the exact bf16
// value of the reference decoder and fed to v_mfma_f32_32x32x16_bf16 against x
// fragments read straight from global memory (x is small and stays in L2).
// A block owns 32 weight rows and all of K; its eight waves each stream one
// eighth of K and the partial sums meet in LDS in a fixed order (no atomics
// on the output, no device-scope fences).
#include "xq_common.h"
#include "xq_lora.h"

namespace xq {

struct SkinnyArgs {
    const bf16_t* x;
    int64_t ldx;
    int32_t M, N, K;
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int32_t group, scale_dtype;
    const float* su_f32;       // [M, r_pad] fp32 sums of x . A^T (unscaled) or NULL
    float su_scale;
    const bf16_t* lora_right;  // [N, r_pad]
    int32_t r_pad;
    const bf16_t* bias;
    bf16_t* y;
    int64_t ldy;
};

// decode 8 consecutive K elements (one MFMA operand) of this lane's row
template <int FMT>
__device__ __forceinline__ bf16x8 decode8(uint32_t w0, uint32_t w1, float s0, float s1) {
    uint32_t o[4];
    if (FMT == XQ_FMT_FP8) {
        f32x2 a = e4m3x2_to_f32(w0, false), b = e4m3x2_to_f32(w0, true);
        f32x2 c = e4m3x2_to_f32(w1, false), d = e4m3x2_to_f32(w1, true);
        o[0] = pack_bf16x2(a[0] * s0, a[1] * s0);
        o[1] = pack_bf16x2(b[0] * s0, b[1] * s0);
        o[2] = pack_bf16x2(c[0] * s0, c[1] * s0);
        o[3] = pack_bf16x2(d[0] * s0, d[1] * s0);
    } else if (FMT == XQ_FMT_INT4) {
        // w0 holds 8 nibbles; fma(nib, s, -8s) == fl((nib-8)*s) up to the sign of zero
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float lo = __builtin_fmaf((float)((w0 >> (8 * i)) & 0xfu), s0, s1);
            float hi = __builtin_fmaf((float)((w0 >> (8 * i + 4)) & 0xfu), s0, s1);
            o[i] = pack_bf16x2(lo, hi);
        }
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

// One block = 32*NT weight rows x the whole K, SK_NW waves each streaming 1/SK_NW of K
// (in-block split-K: no atomics, no fences, fixed summation order).  x fragments are read
// straight from global memory (it is small and L2 resident); rows >= M are never touched.
constexpr int SK_NW = 8;   // waves per block; each streams 1/SK_NW of K

// One block = 32 weight rows x the whole K, SK_NW waves each streaming 1/SK_NW of K
// (in-block split-K: no atomics, no fences, fixed summation order).  A wave fetches its
// codes in batches of 8 KB (all loads of a batch are issued before any is used) and reads
// its x fragments from global memory just in time (x is small and L1/L2 resident).
template <int FMT, int MT>
__global__ void __launch_bounds__(SK_NW * 64) skinny_kernel(SkinnyArgs g) {
    extern __shared__ __attribute__((aligned(16))) float red[];   // [SK_NW waves][MT*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps the K-range loop on scalar branches
    const int fr = lane & 31, fh = lane >> 5;
    const int n0 = blockIdx.x * 32;
    constexpr int EB = FMT == XQ_FMT_FP8 ? 1 : 2;      // elements per byte
    constexpr int NLOAD = FMT == XQ_FMT_FP8 ? 4 : 2;   // 16-byte loads per lane per 128-k chunk
    constexpr int BC = FMT == XQ_FMT_FP8 ? 2 : 4;      // chunks per batch (8 x 16 B per lane)
    const float gsc = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;

    int n = n0 + fr;
    n = n < g.N ? n : g.N - 1;
    const uint8_t* wrow = g.packed + ((int64_t)n * g.K + fh * 64) / EB;
    // Lanes whose row m is >= M read x row 0 instead (no per-lane branches): column m of the
    // product depends only on x row m, and columns >= M are never stored.
    const bf16_t* xg[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i) {
        const int m = i * 32 + fr;
        xg[i] = g.x + (int64_t)(m < g.M ? m : 0) * g.ldx + fh * 64;
    }

    f32x16 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][q] = 0.0f;

    // low-rank operands (last wave only), loaded now so their latency hides under the weight stream
    const bool lora_wave = g.r_pad > 0 && wave == SK_NW - 1;
    bf16x8 lb[4], ls[MT][4];
    if (lora_wave) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks < (g.r_pad >> 4)) {
                lb[ks] = *(const bf16x8*)(g.lora_right + (int64_t)n * g.r_pad + ks * 16 + fh * 8);
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const int m = i * 32 + fr;
                    const float* sp = g.su_f32 + (int64_t)(m < g.M ? m : 0) * g.r_pad + ks * 16 + fh * 8;
                    uint32_t o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = pack_bf16x2(sp[2 * e] * g.su_scale, sp[2 * e + 1] * g.su_scale);
                    u32x4 r = {o[0], o[1], o[2], o[3]};
                    ls[i][ks] = __builtin_bit_cast(bf16x8, r);
                }
            }
        }
    }

    const int ct = g.K >> 7;                                   // 128-element chunks in K
    const int c_begin = (ct * wave) / SK_NW, c_end = (ct * (wave + 1)) / SK_NW;

    for (int c0 = c_begin; c0 < c_end; c0 += BC) {
        u32x4 w[BC][NLOAD];
        float sc[BC];
        // ---- issue every load of the batch
#pragma unroll
        for (int b = 0; b < BC; ++b) {
            if (c0 + b < c_end) {
                const int c = c0 + b, k0 = c * 128 + fh * 64;
#pragma unroll
                for (int i = 0; i < NLOAD; ++i) w[b][i] = *(const u32x4*)(wrow + (int64_t)c * (128 / EB) + i * 16);
                sc[b] = 0.0f;
                if (FMT == XQ_FMT_FP8) sc[b] = ((const float*)g.scales)[(n >> 7) * ((g.K + 127) >> 7) + (k0 >> 7)];
                else if (FMT == XQ_FMT_INT4 && g.group >= 64) sc[b] = load_scale(g.scales, ((int64_t)n * g.K + k0) / g.group, g.scale_dtype);
            }
        }
        // ---- decode + multiply
#pragma unroll
        for (int b = 0; b < BC; ++b) {
            if (c0 + b < c_end) {
                const int c = c0 + b, k0 = c * 128 + fh * 64;
                bf16x8 xf[MT][8];
#pragma unroll
                for (int i = 0; i < MT; ++i)
#pragma unroll
                    for (int t = 0; t < 8; ++t) xf[i][t] = *(const bf16x8*)(xg[i] + c * 128 + t * 8);
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    bf16x8 wf;
                    if (FMT == XQ_FMT_FP8) {
                        wf = decode8<FMT>(w[b][t >> 1][(t & 1) * 2], w[b][t >> 1][(t & 1) * 2 + 1], sc[b], 0.0f);
                    } else if (FMT == XQ_FMT_INT4) {
                        float s = g.group >= 64 ? sc[b] : load_scale(g.scales, ((int64_t)n * g.K + k0 + t * 8) / g.group, g.scale_dtype);
                        wf = decode8<FMT>(w[b][t >> 2][t & 3], 0u, s, -8.0f * s);
                    } else {
                        float s = load_scale(g.scales, ((int64_t)n * g.K + k0 + t * 8) >> 4, g.scale_dtype) * gsc;
                        wf = decode8<FMT>(w[b][t >> 2][t & 3], 0u, s, 0.0f);
                    }
#pragma unroll
                    for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf[i][t], acc[i], 0, 0, 0);
                }
            }
        }
    }

    // ---- low-rank side term: its operands were fetched before the stream started
    if (lora_wave) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks < (g.r_pad >> 4)) {
#pragma unroll
                for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb[ks], ls[i][ks], acc[i], 0, 0, 0);
            }
        }
    }

    // ---- cross-wave reduction through LDS, summed in wave order
    constexpr int R = MT * 16;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) red[(wave * R + i * 16 + q) * 64 + lane] = acc[i][q];
    __syncthreads();
    // quads of 4 consecutive output columns: quad id = (i, q4); wave w takes quads w, w+SK_NW, ...
    for (int quad = wave; quad < MT * 4; quad += SK_NW) {
        const int i = quad >> 2, q4 = quad & 3;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < SK_NW; ++w)
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += red[(w * R + i * 16 + q4 * 4 + e) * 64 + lane];
        const int m = i * 32 + fr, nn = n0 + 8 * q4 + 4 * fh;
        if (m < g.M && nn < g.N) {   // N % 16 == 0: groups of 4 columns are all in or all out
            if (g.bias) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] += bf16_to_f32(g.bias[nn + e]);
            }
            *(u32x2*)(g.y + (int64_t)m * g.ldy + nn) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
    }
}

// partial sums of x . A^T over one 256-wide K range, added with atomics to su_f32 [M, r_pad] (zeroed)
template <int MT>
__global__ void __launch_bounds__(64) skinny_su_kernel(const bf16_t* x, int64_t ldx, int M, int K, const bf16_t* A_bf,
                                                       int r_pad, float* su_f32) {
    const int lane = threadIdx.x, fr = lane & 31, fh = lane >> 5;
    const int kb = blockIdx.x * 256;
    const int nt = (r_pad + 31) >> 5;
    for (int j = 0; j < nt; ++j) {
        const int rrow = j * 32 + fr;
        f32x16 acc[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][q] = 0.0f;
        const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int k = kb; k < kb + 256 && k < K; k += 16) {
            bf16x8 af = rrow < r_pad ? *(const bf16x8*)(A_bf + (int64_t)rrow * K + k + fh * 8) : z;
#pragma unroll
            for (int i = 0; i < MT; ++i) {
                const int m = i * 32 + fr;
                bf16x8 xf = m < M ? *(const bf16x8*)(x + (int64_t)m * ldx + k + fh * 8) : z;
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af, xf, acc[i], 0, 0, 0);   // D[rank][m]
            }
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) {
            const int m = i * 32 + fr;
            if (m >= M) continue;
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int rr = j * 32 + (q & 3) + 4 * fh + 8 * (q >> 2);
                if (rr < r_pad) atomicAdd(su_f32 + (int64_t)m * r_pad + rr, acc[i][q]);
            }
        }
    }
}

static inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }

int64_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int r_pad) {
    return al256(M * (r_pad ? r_pad : 16) * 4) + al256((int64_t)r_pad * K * 2) + al256(N * (int64_t)r_pad * 2) + 256;
}

bool skinny_supported(const xq_weight* w, int64_t M) {
    if (M < 1 || M > 64 || w->num_experts != 1) return false;
    if (w->format != XQ_FMT_FP8 && w->layout != XQ_LAYOUT_FLAT) return false;
    if (w->cols % 128 != 0 || w->cols < 1024 || w->rows % 16 != 0) return false;
    if (w->format == XQ_FMT_INT4 && (w->group % 8 != 0)) return false;
    return true;
}

template <int FMT>
static int launch_skinny_cfg(const SkinnyArgs& g, hipStream_t s) {
    dim3 grid((unsigned)xq_cdiv(g.N, 32));
    if (g.M <= 32) skinny_kernel<FMT, 1><<<grid, SK_NW * 64, (size_t)SK_NW * 16 * 64 * 4, s>>>(g);
    else skinny_kernel<FMT, 2><<<grid, SK_NW * 64, (size_t)SK_NW * 32 * 64 * 4, s>>>(g);
    return XQ_OK;
}

int launch_skinny(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                  int lora_dtype, int r, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, void* workspace,
                  int64_t workspace_bytes, hipStream_t stream) {
    const int64_t N = w->rows, K = w->cols;
    const int rp = r <= 0 ? 0 : ((r + 15) / 16) * 16;
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= skinny_workspace_bytes(M, N, K, rp),
               "xq_linear_fwd: workspace missing, misaligned or too small for the skinny path");
    XQ_REQUIRE(ldx % 8 == 0 && xq_aligned(x, 16) && xq_aligned(w->packed, 16), "xq_linear_fwd: operands must be 16-byte aligned");
    uint8_t* p = (uint8_t*)workspace;
    float* su_f32 = (float*)p; p += al256(M * (rp ? rp : 16) * 4);
    bf16_t* A_bf = (bf16_t*)p; p += al256((int64_t)rp * K * 2);
    bf16_t* Bl = (bf16_t*)p;

    int rc;
    if (rp) {
        if ((rc = launch_zero_fill(su_f32, M * rp * 4, stream))) return rc;
        if ((rc = launch_factor_prep(lora_A, lora_dtype, r, K, false, A_bf, rp, K, 1, stream))) return rc;
        if ((rc = launch_factor_prep(lora_B, lora_dtype, N, r, false, Bl, N, rp, 1, stream))) return rc;
        dim3 sg((unsigned)xq_cdiv(K, 256));
        if (M <= 32) skinny_su_kernel<1><<<sg, 64, 0, stream>>>(x, ldx, (int)M, (int)K, A_bf, rp, su_f32);
        else skinny_su_kernel<2><<<sg, 64, 0, stream>>>(x, ldx, (int)M, (int)K, A_bf, rp, su_f32);
        XQ_CHECK_LAUNCH("skinny_su");
    }
    SkinnyArgs g;
    g.x = x; g.ldx = ldx; g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.group = w->group; g.scale_dtype = w->scale_dtype;
    g.su_f32 = rp ? su_f32 : nullptr; g.su_scale = scaling; g.lora_right = rp ? Bl : nullptr; g.r_pad = rp;
    g.bias = bias; g.y = y; g.ldy = ldy;
    // algorithmic bytes: packed weight + scales + x + y (+ LoRA factors), for the roofline figure
    const double wbytes = (double)xq_packed_bytes_per_expert(w) + (double)xq_scale_bytes_per_expert(w);
    const bool timed = xq_profile_mark_begin(stream, wbytes + 2.0 * M * K + 2.0 * M * N + 4.0 * r * (K + N));
    if (w->format == XQ_FMT_FP8) rc = launch_skinny_cfg<XQ_FMT_FP8>(g, stream);
    else if (w->format == XQ_FMT_INT4) rc = launch_skinny_cfg<XQ_FMT_INT4>(g, stream);
    else rc = launch_skinny_cfg<XQ_FMT_NVFP4>(g, stream);
    if (timed) xq_profile_mark_end(stream);
    if (rc) return rc;
    XQ_CHECK_LAUNCH("skinny_kernel");
    return XQ_OK;
}

}  // namespace xq
