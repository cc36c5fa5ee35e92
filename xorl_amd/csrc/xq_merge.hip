// Merging the LoRA update into the quantized base weight without materialising it:
//
//   W'[n, k] = deq(W)[n, k] + scaling * sum_j B[n, j] * A[j, k]          (W FLAT [N, K])
//
// One block owns a 128 x 128 tile -- exactly one block-fp8 scale block.  It
//   0. issues every load it will need before waiting for any: the tile's packed codes (16-element runs,
//      coalesced: consecutive lanes walk a row) and scales, then its MFMA operands.  All loads are
//      unconditional (indices past the end are clamped, values masked), so the waits count exactly and the
//      codes arrive while the low-rank product is computed;
//   1. computes the tile of the low-rank product on the matrix cores.  The reference multiplies the fp32
//      factors in fp32; here each factor is split into two bf16 terms (hi + lo, 16 significant bits) and the
//      product is the three bf16 MFMA products hi*hi + hi*lo + lo*hi with fp32 accumulation (relative error
//      ~2^-16 per term instead of 2^-9 with plain bf16 factors).  A small launch before it (merge_prep_kernel)
//      splits scaling * B and A^T once into zero-padded bf16 panels in the caller's workspace, laid out so
//      that a tile's rows are one contiguous run of each panel: the tile kernel copies them to LDS with 16-byte
//      pieces and multiplies while its codes are still in flight;
//   2. hands it to the row-contiguous pass through LDS, 64 columns at a time: every thread decodes its runs
//      to the reference decoder's value and adds the update;
//   3a. (publish) rounds to bf16 -- bf16(bf16(deq) + bf16(delta)), the arithmetic of the reference's
//      weight-sync merge -- or writes the fp32 sum; or
//   3b. (requantise, block-fp8) reduces the tile's absmax, derives the new block scale
//      s = max(amax / 448, 1e-12) and writes e4m3(clamp(x / s)) bytes and the scale: decode -> add ->
//      re-encode in one pass over 1 byte per weight each way.
#include "xq_common.h"
#include <atomic>
#include "xq_lora.h"

namespace xq {

constexpr int MG_T = 128;           // tile edge
constexpr int MG_HP = 64 + 4;       // delta half-tile row pitch (floats)

struct MergeArgs {
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int32_t fmt, group, scale_dtype;
    int32_t N, K;
    const void* A;       // [r, K]   } read by merge_prep_kernel only
    const void* B;       // [N, r]   }
    int32_t lora_f32, r, r_pad;
    float scaling;
    const bf16_t* Bh;    // factor panels written by merge_prep_kernel: hi and lo bf16 parts of scaling * B, rows
    const bf16_t* Bl;    // padded to a multiple of 128 ([Npad][r_pad], zero beyond N and r), and of A transposed
    const bf16_t* Ah;    // ([Kpad][r_pad], row = k)
    const bf16_t* Al;
    int32_t mode;        // 0: bf16 out (publish arithmetic), 1: fp32 out, 2: block-fp8 requantise,
                         // 3: absmax of the mode-0 values only, 4 / 5: nvfp4 / nf4 requantise of the mode-0 values,
                         // 6 / 7: int4 requantise of the mode-0 values, 128-element groups along K (6: scale =
                         // bf16(absmax / 7), codes rne(x / scale) in [-7, 7] + 8; 7: the reference's rule, fp32 scales)
    void* out;           // mode 0/1: [N, K]
    uint8_t* packed_out; // mode 2: [N, K] e4m3 bytes    } both may alias the inputs: a block reads its tile and its
    float* scales_out;   // mode 2: [ceil(N/128), ceil(K/128)] } scale before it writes them, and touches no other
                         // mode 5: [N, K/64] fp32; mode 6: [N, K/128] bf16; mode 7: [N, K/128] fp32
    float* amax_out;     // mode 3: one float, zeroed before the launch; receives max |value| over the matrix
    const float* gamax;  // mode 4: the tensor-level amax the scales are derived from (one float on the device)
    uint8_t* codes_out;  // mode 4 / 5: [N, K/2] code pairs     } may alias the inputs (tile-local, read before written);
    uint8_t* bscale_out; // mode 4: [N, K/16] e4m3 block scales } the global scale output may not
    float* gscale_out;   // mode 4: one float
};

// NF4 code of a value already normalised into [-1, 1]: the number of midpoints between neighbouring levels that lie
// strictly below it (ops/quantize/nf4_codec.py:42-64)
__device__ __forceinline__ uint32_t nf4_encode(float v) {
    constexpr float kMid[15] = {(float)-0.8480964004993439, (float)-0.6106329262256622, (float)-0.4599952697753906,
                                (float)-0.3396794348955154, (float)-0.2346074059605598, (float)-0.1379117332398891,
                                (float)-0.0455250181257725, (float)0.0397901497781277,  (float)0.1202552504837513,
                                (float)0.2035212516784668,  (float)0.2920137718319893,  (float)0.3893125355243683,
                                (float)0.5016634166240692,  (float)0.6427869200706482,  (float)0.8614784181118012};
    uint32_t c = 0;
#pragma unroll
    for (int i = 0; i < 15; ++i) c += v > kMid[i] ? 1u : 0u;
    return c;
}

// e2m1 code of a value already scaled into [-6, 6] (ops/quantize/fp4_codec.py:12-19: ties go up in magnitude)
__device__ __forceinline__ uint32_t fp4_encode(float v) {
    const float a = fabsf(v);
    int lo = (int)(a * 2.0f + 0.5f);
    lo = lo > 3 ? 3 : lo;
    const int hi = 4 + (a >= 2.5f) + (a >= 3.5f) + (a >= 5.0f);
    return (uint32_t)(a >= 1.75f ? hi : lo) + (v < 0.0f ? 8u : 0u);
}

// hi/lo bf16 split of the factors, once per call instead of once per tile: Bh/Bl[n][j] from scaling * B[n][j],
// Ah/Al[k][j] from A[j][k] (transposed so that a tile's MFMA operand rows are contiguous 16-byte pieces).
// Rows beyond N / K (up to the next multiple of 128) and ranks beyond r are zero, so the tile kernel reads the
// panels without bounds checks.
__global__ void __launch_bounds__(256) merge_prep_kernel(MergeArgs g, int npad, int kpad) {
    const int rp = g.r_pad;
    const int64_t nb = (int64_t)npad * rp, na = (int64_t)kpad * rp;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool f32 = g.lora_f32 != 0;
    if (idx < nb) {
        const int64_t n = idx / rp;
        const int j = (int)(idx - n * rp);
        float v = 0.0f;
        if (n < g.N && j < g.r) v = g.scaling * (f32 ? ((const float*)g.B)[n * g.r + j] : bf16_to_f32(((const bf16_t*)g.B)[n * g.r + j]));
        const bf16_t hi = to_bf16(v);
        ((bf16_t*)g.Bh)[idx] = hi;
        ((bf16_t*)g.Bl)[idx] = to_bf16(v - bf16_to_f32(hi));
    } else if (idx < nb + na) {
        const int64_t t = idx - nb;           // k fastest: coalesced reads of A's rows
        const int j = (int)(t / kpad);
        const int64_t k = t - (int64_t)j * kpad;
        float v = 0.0f;
        if (k < g.K && j < g.r) v = f32 ? ((const float*)g.A)[(int64_t)j * g.K + k] : bf16_to_f32(((const bf16_t*)g.A)[(int64_t)j * g.K + k]);
        const bf16_t hi = to_bf16(v);
        ((bf16_t*)g.Ah)[k * rp + j] = hi;
        ((bf16_t*)g.Al)[k * rp + j] = to_bf16(v - bf16_to_f32(hi));
    }
}

// REQ: the block-fp8 re-quantise mode (results are held in registers until the tile's absmax is known) and, for an
// int4 weight, the int4 one (held until the row's 128-element group, which is the tile's whole row, is known).
// 512 threads per tile: 32 result registers per thread in that mode, so that two blocks (16 waves) fit a CU.
template <int FMT, int RP, bool REQ>
__global__ void __launch_bounds__(512, 4) merge_kernel(MergeArgs g) {
    asm volatile("" ::"s"(g.packed), "s"(g.scales), "s"(g.global_scale), "s"(g.group), "s"(g.scale_dtype), "s"(g.N), "s"(g.K),
                 "s"(g.Bh), "s"(g.Bl), "s"(g.Ah), "s"(g.Al), "s"(g.mode), "s"(g.out), "s"(g.packed_out), "s"(g.scales_out));
    // (all arguments in scalar registers after one round trip)
    extern __shared__ __attribute__((aligned(16))) uint8_t mg_lds[];
    __shared__ float sh_amax[8];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int k0 = blockIdx.x * MG_T, n0 = blockIdx.y * MG_T;
    constexpr bool FP8 = FMT == XQ_FMT_FP8;
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    // ---- 0a. this tile's rows of the four factor panels -> registers (16-byte pieces, each tile one contiguous
    // run of its panel), issued before the codes so that they can be waited for on their own
    constexpr int FP = RP + 8;                        // LDS row pitch (bf16 elements): fragment reads are conflict free
    constexpr int PPRW = RP / 8;                      // 16-byte pieces per panel row
    constexpr int NP = RP / 8;                        // pieces per thread: 4 tiles x 128 rows x PPRW / 512
    u32x4 fp[NP > 0 ? NP : 1];
    if (RP > 0) {
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = tid + 512 * i, tile = p / (128 * PPRW), q = p % (128 * PPRW);
            const bf16_t* base = tile == 0 ? g.Bh + (int64_t)n0 * RP : tile == 1 ? g.Bl + (int64_t)n0 * RP
                               : tile == 2 ? g.Ah + (int64_t)k0 * RP : g.Al + (int64_t)k0 * RP;
            fp[i] = *(const u32x4*)(base + q * 8);
        }
    }

    // ---- 0b. the tile's codes: run h of this thread = row tid >> 2, columns h*64 + (tid & 3)*16 .. +15
    const int rrow = tid >> 2, rcol = (tid & 3) * 16;
    u32x4 wr[2];                                      // fp8: 16 bytes; 4-bit: 8 bytes (first two words)
    uint32_t sraw[2];                                 // 4-bit: the run's scale (group % 16 == 0), raw
    const bool run_scale = !FP8 && (g.group & 15) == 0;
    float tile_scale = 1.0f;
    if (FP8) tile_scale = ((const float*)g.scales)[(int64_t)blockIdx.y * ((g.K + 127) >> 7) + blockIdx.x];
    const int64_t nrow = n0 + rrow < g.N ? n0 + rrow : g.N - 1;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int k = k0 + h * 64 + rcol < g.K ? k0 + h * 64 + rcol : g.K - 16;   // K % 16 == 0
        if (FP8) wr[h] = *(const u32x4*)(g.packed + nrow * g.K + k);
        else {
            const u32x2 t = *(const u32x2*)(g.packed + ((nrow * g.K + k) >> 1));
            wr[h] = u32x4{t[0], t[1], 0u, 0u};
            const int64_t si = run_scale ? (nrow * g.K + k) / g.group : 0;
            sraw[h] = g.scale_dtype == XQ_SCALE_F32 ? ((const uint32_t*)g.scales)[si]
                    : g.scale_dtype == XQ_SCALE_BF16 ? ((const uint16_t*)g.scales)[si] : g.scales[si];
        }
    }
    const float gs = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;

    float* dt = (float*)mg_lds;   // delta half tile [128][MG_HP] (takes the place of the factor tiles)
    f32x16 acc[2];                // wave (wq, wh): rows wq*32 .. +31, columns wh*64 + j*32 .. +31
    const int wq = wave & 3, wh = wave >> 2, fr = lane & 31, fk = (lane >> 5) * 8;
    if (RP > 0) {
        // ---- 1. factor tiles -> LDS ([tile][128][FP]); the delta tile on the matrix cores while the codes are
        // still in flight
        bf16_t* ft = (bf16_t*)mg_lds;
#pragma unroll
        for (int i = 0; i < NP; ++i) {
            const int p = tid + 512 * i, tile = p / (128 * PPRW), q = p % (128 * PPRW);
            *(u32x4*)(ft + (tile * 128 + q / PPRW) * FP + (q % PPRW) * 8) = fp[i];
        }
        lds_barrier();
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[j][q] = 0.0f;
        const bf16_t* pb = ft + (wq * 32 + fr) * FP + fk;                    // Bh rows of this wave; Bl one tile further
        const bf16_t* pa = ft + (2 * 128 + wh * 64 + fr) * FP + fk;          // Ah rows of this wave's columns; Al one tile further
#pragma unroll
        for (int ks = 0; ks < (RP >> 4); ++ks) {
            const bf16x8 bh = *(const bf16x8*)(pb + ks * 16), bl = *(const bf16x8*)(pb + 128 * FP + ks * 16);
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const bf16x8 ah = *(const bf16x8*)(pa + j * 32 * FP + ks * 16), al = *(const bf16x8*)(pa + (128 + j * 32) * FP + ks * 16);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bl, ah, acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh, al, acc[j], 0, 0, 0);
                acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh, ah, acc[j], 0, 0, 0);
            }
        }
    }

    // ---- 2./3. per 64-column half: delta half tile -> LDS (the four waves that own it), row-contiguous pass
    float m[REQ ? 32 : 1];
    float amax = 0.0f;
    const int64_t n = n0 + rrow;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        if (RP > 0) {
            lds_barrier();   // h = 0: the factor tiles are dead; h = 1: the first half has been read
            if (wh == h) {
                const int rgrp = (lane >> 5) * 4;
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int q = 0; q < 16; ++q) {
                        const int row = wq * 32 + (q & 3) + rgrp + 8 * (q >> 2), col = j * 32 + fr;
                        dt[row * MG_HP + col] = acc[j][q];
                    }
            }
            lds_barrier();
        }
        const int k = k0 + h * 64 + rcol;
        const bool ok = n < g.N && k < g.K;               // K % 16 == 0: runs are all in or all out
        float v[16];
        if (FP8) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const f32x2 lo = e4m3x2_to_f32(wr[h][i], false), hi = e4m3x2_to_f32(wr[h][i], true);
                v[4 * i] = lo[0] * tile_scale; v[4 * i + 1] = lo[1] * tile_scale;
                v[4 * i + 2] = hi[0] * tile_scale; v[4 * i + 3] = hi[1] * tile_scale;
            }
        } else {
            const uint32_t sr = sraw[h];
            const float srun = g.scale_dtype == XQ_SCALE_F32 ? __uint_as_float(sr)
                             : g.scale_dtype == XQ_SCALE_BF16 ? __uint_as_float(sr << 16) : e4m3_to_f32((uint8_t)sr);
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t nib = (wr[h][i >> 3] >> (4 * (i & 7))) & 0xfu;
                // groups that are not multiples of 16 (never with the reference's formats): per-element lookup
                const float sc = run_scale ? srun : load_scale(g.scales, (nrow * g.K + (k < g.K ? k : 0) + i) / g.group, g.scale_dtype);
                v[i] = val4<FMT>(nib, FMT == XQ_FMT_NVFP4 ? sc * gs : sc);
            }
        }
        float x[16];
#pragma unroll
        for (int i = 0; i < 16; i += 4) {
            f32x4 d = {0.0f, 0.0f, 0.0f, 0.0f};
            if (RP > 0) d = *(const f32x4*)(dt + rrow * MG_HP + rcol + i);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float t;
                if (g.mode == 0 || g.mode >= 3 || !FP8) t = bf16_to_f32(to_bf16(bf16_to_f32(to_bf16(v[i + e])) + bf16_to_f32(to_bf16(d[e]))));   // 4-bit decoders return bf16
                else t = v[i + e] + d[e];
                x[i + e] = ok ? t : 0.0f;
            }
        }
        if (REQ) {
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                m[h * 16 + i] = x[i];
                amax = fmaxf(amax, fabsf(x[i]));
            }
        } else if (g.mode == 3) {
#pragma unroll
            for (int i = 0; i < 16; ++i) amax = fmaxf(amax, fabsf(x[i]));
        } else if (g.mode == 4) {
            // one nvfp4 block per run (ops/quantize/nvfp4_quantize.py:25-60,102-111): codes against the raw block
            // amax, block scale = e4m3(amax / global amax * 448)
            if (ok) {
                float bmax = 0.0f;
#pragma unroll
                for (int i = 0; i < 16; ++i) bmax = fmaxf(bmax, fabsf(x[i]));
                bmax = fmaxf(bmax, 1e-12f);
                const float q = 6.0f / bmax;
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    lo |= fp4_encode(__builtin_amdgcn_fmed3f(x[i] * q, -6.0f, 6.0f)) << (4 * i);
                    hi |= fp4_encode(__builtin_amdgcn_fmed3f(x[8 + i] * q, -6.0f, 6.0f)) << (4 * i);
                }
                *(u32x2*)(g.codes_out + ((n * g.K + k) >> 1)) = u32x2{lo, hi};
                const float gm = fmaxf(g.gamax[0], 1e-12f);
                const float bs = __builtin_amdgcn_fmed3f(bmax / gm * 448.0f, -448.0f, 448.0f);
                g.bscale_out[(n * g.K + k) >> 4] = (uint8_t)(__builtin_amdgcn_cvt_pk_fp8_f32(bs, 0.0f, 0u, false) & 0xffu);
            }
        } else if (g.mode == 5) {
            // NF4 (ops/quantize/nf4_quantize.py:20-56): a 64-element group is the four runs of four neighbouring lanes;
            // scale = max(absmax, 1e-12), code = encode(clamp(x * (1 / scale), +-1))
            float bmax = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) bmax = fmaxf(bmax, fabsf(x[i]));
            bmax = fmaxf(bmax, __shfl_xor(bmax, 1, 64));
            bmax = fmaxf(bmax, __shfl_xor(bmax, 2, 64));
            const float sc = fmaxf(bmax, 1e-12f), inv = 1.0f / sc;
            if (ok) {
                uint32_t lo = 0, hi = 0;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    lo |= nf4_encode(__builtin_amdgcn_fmed3f(x[i] * inv, -1.0f, 1.0f)) << (4 * i);
                    hi |= nf4_encode(__builtin_amdgcn_fmed3f(x[8 + i] * inv, -1.0f, 1.0f)) << (4 * i);
                }
                *(u32x2*)(g.codes_out + ((n * g.K + k) >> 1)) = u32x2{lo, hi};
                if ((tid & 3) == 0) g.scales_out[(n * g.K + k) >> 6] = sc;
            }
        } else if (ok) {
            if (g.mode == 0) {
                bf16_t* o = (bf16_t*)g.out + n * g.K + k;
                uint32_t pk[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) pk[i] = pack_bf16x2(x[2 * i], x[2 * i + 1]);
                *(u32x4*)o = u32x4{pk[0], pk[1], pk[2], pk[3]};
                *(u32x4*)(o + 8) = u32x4{pk[4], pk[5], pk[6], pk[7]};
            } else {
                float* o = (float*)g.out + n * g.K + k;
#pragma unroll
                for (int i = 0; i < 4; ++i) *(f32x4*)(o + 4 * i) = f32x4{x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]};
            }
        }
    }
    if constexpr (REQ && FMT == XQ_FMT_INT4) {
        // ---- 3a. int4, one group per tile row: the four lanes of a row hold its 128 values
        float ga = amax;
        ga = fmaxf(ga, __shfl_xor(ga, 1, 64));
        ga = fmaxf(ga, __shfl_xor(ga, 2, 64));
        if (n >= g.N) return;
        const int64_t gi = (n * g.K + k0) >> 7;
        uint32_t pk[4] = {0u, 0u, 0u, 0u};
        if (g.mode == 6) {
            // scale = bf16(absmax / 7); code = clamp(rne(x / scale), -7, 7) + 8, all zero codes (8) for a zero group
            const bf16_t sb = to_bf16(ga / 7.0f);
            const float sc = bf16_to_f32(sb);
            if ((tid & 3) == 0) ((bf16_t*)g.scales_out)[gi] = sb;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const float q = sc > 0.0f ? __builtin_amdgcn_fmed3f(__builtin_rintf(m[i] / sc), -7.0f, 7.0f) : 0.0f;
                pk[i >> 3] |= (uint32_t)((int)q + 8) << (4 * (i & 7));
            }
        } else {
            // ops/quantize/int4_quantize.py:12-41: scale = max(absmax, 1e-12) * (2/15); code = clamp(trunc(x * (1 / scale)
            // + 8.5), 0, 15) with the product and the sum rounded separately
            const float sc = fmaxf(ga, 1e-12f) * (float)(2.0 / 15.0), inv = 1.0f / sc;
            if ((tid & 3) == 0) g.scales_out[gi] = sc;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const int q = (int)__fadd_rn(__fmul_rn(m[i], inv), 8.5f);
                pk[i >> 3] |= (uint32_t)(q < 0 ? 0 : q > 15 ? 15 : q) << (4 * (i & 7));
            }
        }
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int k = k0 + h * 64 + rcol;
            if (k < g.K) *(u32x2*)(g.codes_out + ((n * g.K + k) >> 1)) = u32x2{pk[2 * h], pk[2 * h + 1]};
        }
        return;
    }
    if (!REQ) {
        if (g.mode == 3) {       // tile absmax -> one atomic per block (values are non-negative: integer order = float order)
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
            if (lane == 0) sh_amax[wave] = amax;
            __syncthreads();
            if (tid == 0) {
                float t = 0.0f;
                for (int i = 0; i < 8; ++i) t = fmaxf(t, sh_amax[i]);
                atomicMax((unsigned int*)g.amax_out, __float_as_uint(t));
            }
        } else if (g.mode == 4 && tid == 0 && blockIdx.x == 0 && blockIdx.y == 0) {
            // global scale = amax / 6 / 448 in the quantizer's operation order
            g.gscale_out[0] = fmaxf(g.gamax[0], 1e-12f) * (1.0f / 6.0f) / 448.0f;
        }
        return;
    }
    // ---- 3b. block absmax -> new scale -> e4m3 bytes
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) sh_amax[wave] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(fmaxf(sh_amax[0], sh_amax[1]), fmaxf(sh_amax[2], sh_amax[3])),
                 fmaxf(fmaxf(sh_amax[4], sh_amax[5]), fmaxf(sh_amax[6], sh_amax[7])));
    const float s = fmaxf(amax / 448.0f, 1e-12f);
    // one division per block; x * (1/s) is within 1.5 ulp of x / s, far inside an e4m3 rounding interval except
    // for quotients within that distance of a rounding boundary
    const float rs = 1.0f / s;
    if (tid == 0) g.scales_out[(int64_t)blockIdx.y * gridDim.x + blockIdx.x] = s;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int k = k0 + h * 64 + rcol;
        if (!(n < g.N && k < g.K)) continue;
        uint32_t pk[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float y[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) y[e] = __builtin_amdgcn_fmed3f(m[h * 16 + 4 * i + e] * rs, -448.0f, 448.0f);
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
    return in + (mode == 0 ? 2.0 * n : mode == 1 ? 4.0 * n : mode == 3 ? 0.0 : in);
}

template <int FMT, int RP, bool REQ>
static int launch_merge_one(const MergeArgs& g, dim3 grid, hipStream_t s, const char* who) {
    // LDS: the four factor tiles, then the delta half tile in their place
    constexpr size_t lds_f = (size_t)4 * MG_T * (RP + 8) * 2, lds_d = (size_t)MG_T * MG_HP * 4;
    constexpr size_t lds = RP == 0 ? 16 : (lds_f > lds_d ? lds_f : lds_d);
    static std::atomic<bool> attr_set{false};   // per instantiation; the attribute call is idempotent: a race only repeats it
    if (!attr_set && lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)merge_kernel<FMT, RP, REQ>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            xq_set_error("%s: cannot raise the dynamic LDS limit: %s", who, hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    merge_kernel<FMT, RP, REQ><<<grid, 512, lds, s>>>(g);
    return XQ_OK;
}

template <int FMT, bool REQ>
static int launch_merge_fmt(const MergeArgs& g, dim3 grid, hipStream_t s, const char* who) {
    switch (g.r_pad) {
        case 0: return launch_merge_one<FMT, 0, REQ>(g, grid, s, who);
        case 16: return launch_merge_one<FMT, 16, REQ>(g, grid, s, who);
        case 32: return launch_merge_one<FMT, 32, REQ>(g, grid, s, who);
        case 48: return launch_merge_one<FMT, 48, REQ>(g, grid, s, who);
        default: return launch_merge_one<FMT, 64, REQ>(g, grid, s, who);
    }
}

static int64_t merge_ws_bytes(int64_t N, int64_t K, int r) {
    const int64_t rp = r <= 0 ? 0 : ((r + 15) / 16) * 16;
    return 256 + 4 * (xq_cdiv(N, MG_T) + xq_cdiv(K, MG_T)) * MG_T * rp;   // four bf16 panels
}

extern "C" int64_t xq_merge_workspace_bytes(int64_t N, int64_t K, int r) { return merge_ws_bytes(N, K, r); }

struct Nvfp4Out {      // outputs of modes 3 and 4
    float* amax_out = nullptr;
    const float* gamax = nullptr;
    uint8_t* codes_out = nullptr;
    uint8_t* bscale_out = nullptr;
    float* gscale_out = nullptr;
};

static int launch_merge(const xq_weight* w, const void* A, const void* B, int lora_dtype, int r, float scaling, int mode,
                        void* out, void* packed_out, float* scales_out, void* workspace, int64_t workspace_bytes,
                        hipStream_t stream, const char* who, const Nvfp4Out& nv = Nvfp4Out()) {
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
    g.amax_out = nv.amax_out; g.gamax = nv.gamax; g.codes_out = nv.codes_out; g.bscale_out = nv.bscale_out; g.gscale_out = nv.gscale_out;
    const int64_t npad = xq_cdiv(w->rows, MG_T) * MG_T, kpad = xq_cdiv(w->cols, MG_T) * MG_T;
    g.Bh = g.Bl = g.Ah = g.Al = nullptr;
    if (g.r_pad > 0) {
        XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= merge_ws_bytes(w->rows, w->cols, r),
                   "%s: workspace missing, misaligned or smaller than xq_merge_workspace_bytes()", who);
        bf16_t* p = (bf16_t*)workspace;
        g.Bh = p; g.Bl = p + npad * g.r_pad; g.Ah = p + 2 * npad * g.r_pad; g.Al = g.Ah + kpad * g.r_pad;
    }
    dim3 grid((unsigned)xq_cdiv(w->cols, MG_T), (unsigned)xq_cdiv(w->rows, MG_T));
    const bool timed = xq_profile_mark_begin(stream, merge_bytes(w, mode));
    if (g.r_pad > 0)
        merge_prep_kernel<<<dim3((unsigned)xq_cdiv((npad + kpad) * g.r_pad, 256)), 256, 0, stream>>>(g, (int)npad, (int)kpad);
    if (w->format == XQ_FMT_FP8) rc = mode == 2 ? launch_merge_fmt<XQ_FMT_FP8, true>(g, grid, stream, who)
                                                : launch_merge_fmt<XQ_FMT_FP8, false>(g, grid, stream, who);
    else if (w->format == XQ_FMT_INT4) rc = mode >= 6 ? launch_merge_fmt<XQ_FMT_INT4, true>(g, grid, stream, who)
                                                      : launch_merge_fmt<XQ_FMT_INT4, false>(g, grid, stream, who);
    else if (w->format == XQ_FMT_NF4) rc = launch_merge_fmt<XQ_FMT_NF4, false>(g, grid, stream, who);
    else rc = launch_merge_fmt<XQ_FMT_NVFP4, false>(g, grid, stream, who);
    if (timed) xq_profile_mark_end(stream);
    if (rc) return rc;
    XQ_CHECK_LAUNCH(who);
    return XQ_OK;
}

extern "C" int xq_merge_dense(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                              float scaling, void* out, int out_dtype, void* workspace, int64_t workspace_bytes,
                              void* stream) {
    XQ_REQUIRE(out_dtype == XQ_DT_BF16 || out_dtype == XQ_DT_F32, "xq_merge_dense: bad out_dtype");
    XQ_REQUIRE(out && xq_aligned(out, 16), "xq_merge_dense: out is NULL or not 16-byte aligned");
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, out_dtype == XQ_DT_BF16 ? 0 : 1, out, nullptr, nullptr,
                        workspace, workspace_bytes, (hipStream_t)stream, "xq_merge_dense");
}

extern "C" int xq_merge_requant_fp8(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                                    float scaling, void* packed_out, float* scales_out, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
    XQ_REQUIRE(w && w->format == XQ_FMT_FP8, "xq_merge_requant_fp8: the weight must be block_fp8");
    XQ_REQUIRE(packed_out && scales_out && xq_aligned(packed_out, 16), "xq_merge_requant_fp8: NULL or misaligned output");
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, 2, nullptr, packed_out, scales_out, workspace, workspace_bytes,
                        (hipStream_t)stream, "xq_merge_requant_fp8");
}

extern "C" int xq_merge_amax(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                             float* amax_out, void* workspace, int64_t workspace_bytes, void* stream) {
    XQ_REQUIRE(amax_out, "xq_merge_amax: amax_out is NULL");
    int rc = launch_zero_fill(amax_out, 4, (hipStream_t)stream);
    if (rc) return rc;
    Nvfp4Out nv;
    nv.amax_out = amax_out;
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, 3, nullptr, nullptr, nullptr, workspace, workspace_bytes,
                        (hipStream_t)stream, "xq_merge_amax", nv);
}

extern "C" int xq_merge_requant_nvfp4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                                      float scaling, const float* global_amax, void* codes_out, void* block_scales_out,
                                      float* global_scale_out, void* workspace, int64_t workspace_bytes, void* stream) {
    XQ_REQUIRE(w && w->format == XQ_FMT_NVFP4 && w->group == 16, "xq_merge_requant_nvfp4: the weight must be nvfp4 with 16-element blocks");
    XQ_REQUIRE(global_amax && codes_out && block_scales_out && global_scale_out && xq_aligned(codes_out, 8),
               "xq_merge_requant_nvfp4: NULL or misaligned output");
    XQ_REQUIRE((const void*)global_scale_out != (const void*)w->global_scale,
               "xq_merge_requant_nvfp4: the new global scale may not overwrite the one the kernel decodes with");
    Nvfp4Out nv;
    nv.gamax = global_amax; nv.codes_out = (uint8_t*)codes_out; nv.bscale_out = (uint8_t*)block_scales_out; nv.gscale_out = global_scale_out;
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, 4, nullptr, nullptr, nullptr, workspace, workspace_bytes,
                        (hipStream_t)stream, "xq_merge_requant_nvfp4", nv);
}

extern "C" int xq_merge_requant_int4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                                     float scaling, int symmetric, void* codes_out, void* scales_out, void* workspace,
                                     int64_t workspace_bytes, void* stream) {
    XQ_REQUIRE(w && w->format == XQ_FMT_INT4 && w->layout == XQ_LAYOUT_FLAT && w->group == 128 && w->cols % 128 == 0,
               "xq_merge_requant_int4: the weight must be flat int4 with 128-element groups and in_features %% 128 == 0");
    XQ_REQUIRE(codes_out && scales_out && xq_aligned(codes_out, 8) && xq_aligned(scales_out, 4),
               "xq_merge_requant_int4: NULL or misaligned output");
    Nvfp4Out nv;
    nv.codes_out = (uint8_t*)codes_out;
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, symmetric ? 6 : 7, nullptr, nullptr, (float*)scales_out,
                        workspace, workspace_bytes, (hipStream_t)stream, "xq_merge_requant_int4", nv);
}

extern "C" int xq_merge_requant_nf4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                                    float scaling, void* codes_out, float* scales_out, void* workspace,
                                    int64_t workspace_bytes, void* stream) {
    XQ_REQUIRE(w && w->format == XQ_FMT_NF4 && w->group == 64 && w->scale_dtype == XQ_SCALE_F32 && w->cols % 64 == 0,
               "xq_merge_requant_nf4: the weight must be NF4 with fp32 scales per 64 elements and in_features %% 64 == 0");
    XQ_REQUIRE(codes_out && scales_out && xq_aligned(codes_out, 8), "xq_merge_requant_nf4: NULL or misaligned output");
    Nvfp4Out nv;
    nv.codes_out = (uint8_t*)codes_out;
    return launch_merge(w, lora_A, lora_B, lora_dtype, r, scaling, 5, nullptr, nullptr, scales_out, workspace, workspace_bytes,
                        (hipStream_t)stream, "xq_merge_requant_nf4", nv);
}
