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
// fragments.  x is small and L2 resident, but every block needs all of it: it is
// fetched with coalesced 16-byte loads (16 lanes per 256-byte row piece) and turned
// into operand fragments through a wave-private, padded LDS tile -- per-lane
// row-strided loads of x would cost more address-unit cycles than the whole weight
// stream.
// A block owns 32 weight rows and all of K; its NW waves (8, or 4 when there are
// more slabs than CUs) each stream 1/NW of K and the partial sums meet in LDS
// in a fixed order (no atomics, no device-scope fences: deterministic).  Loads are
// issued a whole batch at a time -- packed codes, scales and the x fragments of
// the batch together -- into one of two register sets, so the next batch is in
// flight while the current one is decoded and multiplied.
// The low-rank term needs one small launch before it: su = x . A^T (fp32), one
// block whose 16 waves split K; both kernels read the LoRA factors in their own
// dtype (fp32 or bf16), so nothing is repacked or zeroed per call.
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
    const float* su_part;      // [su_parts][M, r_pad] fp32 partial sums of x . A^T (unscaled) or NULL
    int32_t su_parts;
    float su_scale;
    const void* lora_B;        // [N, r] fp32 or bf16
    int32_t lora_f32, r, r_pad;
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

// 8 consecutive LoRA factor entries (fp32 or bf16 storage) -> one MFMA operand; entries at or
// beyond `limit` (counted from the first) are zero
__device__ __forceinline__ bf16x8 factor_frag(const void* base, int64_t idx, bool f32, int limit) {
    uint32_t o[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float lo = 0.0f, hi = 0.0f;
        if (2 * e < limit) lo = f32 ? ((const float*)base)[idx + 2 * e] : bf16_to_f32(((const bf16_t*)base)[idx + 2 * e]);
        if (2 * e + 1 < limit) hi = f32 ? ((const float*)base)[idx + 2 * e + 1] : bf16_to_f32(((const bf16_t*)base)[idx + 2 * e + 1]);
        o[e] = pack_bf16x2(lo, hi);
    }
    u32x4 r = {o[0], o[1], o[2], o[3]};
    return __builtin_bit_cast(bf16x8, r);
}

// One block = 32 weight rows x the whole K, NW waves each streaming 1/NW of K (in-block
// split-K: no atomics, no fences, fixed summation order).  x fragments are read from global
// memory (coalesced, see the top of the file) together with the codes of the same batch.
template <int FMT, int MT, int NW>
__global__ void __launch_bounds__(NW * 64) skinny_kernel(SkinnyArgs g) {
    extern __shared__ __attribute__((aligned(16))) float red[];   // [NW waves][MT*16 regs][64 lanes]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps the K-range loop on scalar branches
    const int fr = lane & 31, fh = lane >> 5;
    const int n0 = blockIdx.x * 32;
    constexpr int EB = FMT == XQ_FMT_FP8 ? 1 : 2;      // elements per byte
    constexpr int NLOAD = FMT == XQ_FMT_FP8 ? 4 : 2;   // 16-byte loads per lane per 128-k chunk
    constexpr int BC = 2 / MT;                         // chunks per batch (per register set)
    constexpr int NSC = FMT == XQ_FMT_NVFP4 ? 4 : 1;   // scale registers per chunk
    const float gsc = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;
    // int4 groups shorter than a lane's 64-element run are looked up per 8 elements at use
    const bool int4_small_group = FMT == XQ_FMT_INT4 && g.group < 64;

    int n = n0 + fr;
    n = n < g.N ? n : g.N - 1;
    const uint8_t* wrow = g.packed + ((int64_t)n * g.K + fh * 64) / EB;
    // x chunk tile of this wave: [MT*32 rows][128 k] bf16, rows padded to 272 B so that the 16 lanes
    // of a b128 read phase (consecutive rows, same column piece) fall on distinct banks.  Rows >= M are
    // never written: they feed only output columns >= M, which are never stored.
    constexpr int XP = 136;                                     // row pitch in bf16 elements
    bf16_t* xs = (bf16_t*)red + wave * (MT * 32 * XP);
    const int xrow = lane >> 4, xpiece = lane & 15;             // coalesced fetch: 4 rows x 16 pieces per instruction
    const bf16_t* xg = g.x + (int64_t)xrow * g.ldx + xpiece * 8;
    const int64_t xstep = 4 * g.ldx;
    const int mrows = g.M;

    f32x16 acc[MT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[i][q] = 0.0f;

    const int ct = g.K >> 7;                                   // 128-element chunks in K
    const int c_begin = (ct * wave) / NW, c_end = (ct * (wave + 1)) / NW;

    struct Batch {
        u32x4 w[BC][NLOAD];
        uint32_t sc[BC][NSC];
        u32x4 xr[BC][MT * 8];
    };
    auto issue = [&](Batch& B, int c0) {
#pragma unroll
        for (int b = 0; b < BC; ++b) {
            if (c0 + b < c_end) {
                const int c = c0 + b, k0 = c * 128 + fh * 64;
#pragma unroll
                for (int i = 0; i < NLOAD; ++i) B.w[b][i] = *(const u32x4*)(wrow + (int64_t)c * (128 / EB) + i * 16);
                if (FMT == XQ_FMT_FP8) B.sc[b][0] = ((const uint32_t*)g.scales)[(n >> 7) * ((g.K + 127) >> 7) + (k0 >> 7)];
                else if (FMT == XQ_FMT_INT4) {
                    if (!int4_small_group) {
                        const int64_t si = ((int64_t)n * g.K + k0) / g.group;
                        B.sc[b][0] = g.scale_dtype == XQ_SCALE_F32 ? ((const uint32_t*)g.scales)[si] : ((const uint16_t*)g.scales)[si];
                    }
                } else {
                    const int64_t si = ((int64_t)n * g.K + k0) >> 4;   // 4 scales of the 64-element run
                    if (g.scale_dtype == XQ_SCALE_E4M3) B.sc[b][0] = *(const uint32_t*)(g.scales + si);
                    else {
                        const u32x4 t = *(const u32x4*)((const float*)g.scales + si);
#pragma unroll
                        for (int j = 0; j < NSC; ++j) B.sc[b][j] = t[j];
                    }
                }
#pragma unroll
                for (int j = 0; j < MT * 8; ++j)
                    if (j * 4 + xrow < mrows) B.xr[b][j] = *(const u32x4*)(xg + j * xstep + c * 128);   // lanes of rows >= M keep stale data
            }
        }
    };
    auto compute = [&](Batch& B, int c0) {
#pragma unroll
        for (int b = 0; b < BC; ++b) {
            if (c0 + b < c_end) {
                const int c = c0 + b, k0 = c * 128 + fh * 64;
                // x tile -> LDS (LDS operations of one wave execute in order: the previous chunk's fragment
                // reads are ahead of these writes)
#pragma unroll
                for (int j = 0; j < MT * 8; ++j)
                    if (j * 4 < mrows) *(u32x4*)(xs + (j * 4 + xrow) * XP + xpiece * 8) = B.xr[b][j];
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    bf16x8 wf;
                    if (FMT == XQ_FMT_FP8) {
                        wf = decode8<FMT>(B.w[b][t >> 1][(t & 1) * 2], B.w[b][t >> 1][(t & 1) * 2 + 1], __uint_as_float(B.sc[b][0]), 0.0f);
                    } else if (FMT == XQ_FMT_INT4) {
                        float s;
                        if (int4_small_group) s = load_scale(g.scales, ((int64_t)n * g.K + k0 + t * 8) / g.group, g.scale_dtype);
                        else s = g.scale_dtype == XQ_SCALE_F32 ? __uint_as_float(B.sc[b][0]) : __uint_as_float(B.sc[b][0] << 16);
                        wf = decode8<FMT>(B.w[b][t >> 2][t & 3], 0u, s, -8.0f * s);
                    } else {
                        float s;
                        if (g.scale_dtype == XQ_SCALE_E4M3) s = e4m3_to_f32((uint8_t)(B.sc[b][0] >> (8 * (t >> 1))));
                        else s = __uint_as_float(B.sc[b][(t >> 1) % NSC]);
                        wf = decode8<FMT>(B.w[b][t >> 2][t & 3], 0u, s * gsc, 0.0f);
                    }
#pragma unroll
                    for (int i = 0; i < MT; ++i) {
                        const bf16x8 xf = *(const bf16x8*)(xs + (i * 32 + fr) * XP + fh * 64 + t * 8);
                        acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc[i], 0, 0, 0);
                    }
                }
            }
        }
    };

    // two register sets: the next batch is in flight while the current one is multiplied
    Batch B0, B1;
    int c = c_begin;
    if (c < c_end) issue(B0, c);

    // ---- low-rank side term (last wave), under the latency of the first batch: acc = (s * su) . B^T with
    // su = x . A^T summed from skinny_su_kernel's parts
    if (g.r_pad > 0 && wave == NW - 1) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            if (ks < (g.r_pad >> 4)) {
                const int j0 = ks * 16 + fh * 8;   // first rank index of this lane's 8
                const bf16x8 lb = factor_frag(g.lora_B, (int64_t)n * g.r + j0, g.lora_f32 != 0, g.r - j0);
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const int m = i * 32 + fr;
                    const float* sp = g.su_part + (int64_t)(m < g.M ? m : 0) * g.r_pad + j0;
                    f32x4 s0 = {0.0f, 0.0f, 0.0f, 0.0f}, s1 = s0;
#pragma unroll 4
                    for (int kb = 0; kb < g.su_parts; ++kb) {   // fixed order
                        s0 += *(const f32x4*)(sp + (int64_t)kb * g.M * g.r_pad);
                        s1 += *(const f32x4*)(sp + (int64_t)kb * g.M * g.r_pad + 4);
                    }
                    uint32_t o[4];
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        o[e] = pack_bf16x2(s0[2 * e] * g.su_scale, s0[2 * e + 1] * g.su_scale);
                        o[2 + e] = pack_bf16x2(s1[2 * e] * g.su_scale, s1[2 * e + 1] * g.su_scale);
                    }
                    u32x4 r = {o[0], o[1], o[2], o[3]};
                    acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(lb, __builtin_bit_cast(bf16x8, r), acc[i], 0, 0, 0);
                }
            }
        }
    }

    while (c < c_end) {
        if (c + BC < c_end) issue(B1, c + BC);
        compute(B0, c);
        c += BC;
        if (c >= c_end) break;
        if (c + BC < c_end) issue(B0, c + BC);
        compute(B1, c);
        c += BC;
    }

    // ---- cross-wave reduction through LDS, summed in wave order (the x tiles are dead by now)
    constexpr int R = MT * 16;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 16; ++q) red[(wave * R + i * 16 + q) * 64 + lane] = acc[i][q];
    __syncthreads();
    // quads of 4 consecutive output columns: quad id = (i, q4); wave w takes quads w, w+NW, ...
    for (int quad = wave; quad < MT * 4; quad += NW) {
        const int i = quad >> 2, q4 = quad & 3;
        float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int w = 0; w < NW; ++w)
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

// Partial sums of su = x[M, K] . A[r, K]^T (fp32, unscaled): block kb covers K range
// [kb*SU_KB, (kb+1)*SU_KB) with its 8 waves (one eighth each, summed through LDS in wave order) and
// writes part[kb][M][r_pad]; columns r..r_pad-1 are zero.  skinny_kernel adds the parts in block
// order, so the low-rank term is deterministic and needs no zeroed buffer and no atomics.
constexpr int SU_KB = 512, SU_NW = 8;
template <int MT>
__global__ void __launch_bounds__(SU_NW * 64) skinny_su_kernel(const bf16_t* x, int64_t ldx, int M, int K, const void* A,
                                                              int a_f32, int r, int r_pad, float* part) {
    extern __shared__ __attribute__((aligned(16))) float red[];   // [SU_NW][MT*16][64]
    const int tid = threadIdx.x, lane = tid & 63, fr = lane & 31, fh = lane >> 5;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int kb0 = blockIdx.x * SU_KB;
    constexpr int SPW = SU_KB / 16 / SU_NW;   // k16 steps per wave
    float* out = part + (int64_t)blockIdx.x * M * r_pad;
    const int nt = (r_pad + 31) >> 5;
    const bf16x8 z = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = 0; j < nt; ++j) {
        const int rrow = j * 32 + fr;
        const bool rvalid = rrow < r;
        f32x16 acc[MT];
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][q] = 0.0f;
#pragma unroll
        for (int s0 = 0; s0 < SPW; s0 += 4) {
            bf16x8 af[4], xf[MT][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {     // the loads of four steps are issued together
                const int kk = kb0 + (wave * SPW + s0 + u) * 16;
                const bool kvalid = kk < K;   // wave-uniform (K % 16 == 0)
                const int k = kk + fh * 8;
                af[u] = kvalid ? factor_frag(A, (int64_t)(rvalid ? rrow : 0) * K + k, a_f32 != 0, rvalid ? 8 : 0) : z;
#pragma unroll
                for (int i = 0; i < MT; ++i) {
                    const int m = i * 32 + fr;
                    xf[i][u] = kvalid ? *(const bf16x8*)(x + (int64_t)(m < M ? m : 0) * ldx + k) : z;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u)
#pragma unroll
                for (int i = 0; i < MT; ++i) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[u], xf[i][u], acc[i], 0, 0, 0);   // D[rank][m]
        }
        constexpr int R = MT * 16;
        __syncthreads();   // the previous rank tile's sums have been read
#pragma unroll
        for (int i = 0; i < MT; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) red[(wave * R + i * 16 + q) * 64 + lane] = acc[i][q];
        __syncthreads();
        for (int idx = wave; idx < R; idx += SU_NW) {   // register idx = (i, q) of every lane
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < SU_NW; ++w) v += red[(w * R + idx) * 64 + lane];
            const int i = idx >> 4, q = idx & 15;
            const int m = i * 32 + fr, rr = j * 32 + (q & 3) + 4 * fh + 8 * (q >> 2);
            if (m < M && rr < r_pad) out[(int64_t)m * r_pad + rr] = v;
        }
    }
}

static inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }

int64_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int r_pad) {
    (void)N;
    return al256(xq_cdiv(K, SU_KB) * M * (r_pad ? r_pad : 16) * 4) + 256;
}

bool skinny_supported(const xq_weight* w, int64_t M) {
    if (M < 1 || M > 64 || w->num_experts != 1) return false;
    if (w->format == XQ_FMT_NF4) return false;   // nf4 takes the tile kernels
    if (w->format != XQ_FMT_FP8 && w->layout != XQ_LAYOUT_FLAT) return false;
    if (w->cols % 128 != 0 || w->cols < 1024 || w->rows % 16 != 0) return false;
    if (w->format == XQ_FMT_INT4 && (w->group % 8 != 0)) return false;
    return true;
}

template <int FMT, int MT, int NW>
static int launch_skinny_one(const SkinnyArgs& g, dim3 grid, hipStream_t s) {
    // LDS: the wave-private x tiles (MT*32 rows of 272 B per wave); the reduction buffer reuses them
    constexpr size_t lds = (size_t)NW * MT * 32 * 136 * 2;
    static_assert(lds >= (size_t)NW * MT * 16 * 64 * 4, "reduction buffer must fit in the x tiles");
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)skinny_kernel<FMT, MT, NW>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) {
            xq_set_error("xq_linear_fwd: cannot raise the dynamic LDS limit: %s", hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    skinny_kernel<FMT, MT, NW><<<grid, NW * 64, lds, s>>>(g);
    return XQ_OK;
}

template <int FMT>
static int launch_skinny_cfg(const SkinnyArgs& g, hipStream_t s) {
    dim3 grid((unsigned)xq_cdiv(g.N, 32));
    // more slabs than CUs: 4 waves per slab so that two blocks share a CU; else 8 waves per slab
    const bool many = grid.x > 256;
    if (g.M <= 32) return many ? launch_skinny_one<FMT, 1, 4>(g, grid, s) : launch_skinny_one<FMT, 1, 8>(g, grid, s);
    return many ? launch_skinny_one<FMT, 2, 4>(g, grid, s) : launch_skinny_one<FMT, 2, 8>(g, grid, s);
}

int launch_skinny(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                  int lora_dtype, int r, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, void* workspace,
                  int64_t workspace_bytes, hipStream_t stream) {
    const int64_t N = w->rows, K = w->cols;
    const int rp = r <= 0 ? 0 : ((r + 15) / 16) * 16;
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= skinny_workspace_bytes(M, N, K, rp),
               "xq_linear_fwd: workspace missing, misaligned or too small for the skinny path");
    XQ_REQUIRE(ldx % 8 == 0 && xq_aligned(x, 16) && xq_aligned(w->packed, 16), "xq_linear_fwd: operands must be 16-byte aligned");
    XQ_REQUIRE(rp == 0 || xq_aligned(lora_A, 4) && xq_aligned(lora_B, 4), "xq_linear_fwd: LoRA factors must be 4-byte aligned");
    float* su_part = (float*)workspace;
    const int su_parts = (int)xq_cdiv(K, SU_KB);

    int rc;
    if (rp) {
        const int f32 = lora_dtype == XQ_DT_F32;
        if (M <= 32) skinny_su_kernel<1><<<dim3(su_parts), SU_NW * 64, (size_t)SU_NW * 16 * 64 * 4, stream>>>(x, ldx, (int)M, (int)K, lora_A, f32, r, rp, su_part);
        else skinny_su_kernel<2><<<dim3(su_parts), SU_NW * 64, (size_t)SU_NW * 32 * 64 * 4, stream>>>(x, ldx, (int)M, (int)K, lora_A, f32, r, rp, su_part);
        XQ_CHECK_LAUNCH("skinny_su");
    }
    SkinnyArgs g;
    g.x = x; g.ldx = ldx; g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.group = w->group; g.scale_dtype = w->scale_dtype;
    g.su_part = rp ? su_part : nullptr; g.su_parts = su_parts; g.su_scale = scaling; g.lora_B = rp ? lora_B : nullptr;
    g.lora_f32 = lora_dtype == XQ_DT_F32; g.r = r; g.r_pad = rp;
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
