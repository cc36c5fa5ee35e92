// Generic fused dequant-GEMM tile kernel (all formats, both layouts, both
// contraction directions, dense and grouped).
//
//   C[rows, Nout] = A[rows, Kc] . Wop  (+ su[rows, r] . Lr[Nout, r]^T) (+ bias)
//
// W is stored [wrows, wcols] (decoded shape).  CONTRACT_COLS = true contracts
// along W's columns (Wop[kc][n] = W[n][kc]; Nout = wrows, Kc = wcols),
// false contracts along its rows (Wop[kc][n] = W[kc][n]; Nout = wcols,
// Kc = wrows).  The packed tile is fetched with 16-byte (8-byte for 4-bit
// FLAT) loads, decoded in registers to the exact bf16 value the reference
// decoder produces, and written to LDS in MFMA operand order ([n][kc], kc
// contiguous); A goes global -> registers -> LDS.  256 threads = 4 waves in a
// 2x2 grid, each wave a 64x64 sub-tile of 2x2 v_mfma_f32_32x32x16_bf16.
#pragma once

#include "xq_common.h"

namespace xq {

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDS_PITCH = BK + 8;  // bf16 elements per LDS row (144 B: conflict-free b128 fragment reads)

struct TileArgs {
    const bf16_t* A;
    int64_t lda;
    bf16_t* C;
    int64_t ldc;
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int64_t packed_stride, scale_stride;  // bytes per expert
    int32_t wrows, wcols;                 // decoded W shape
    int32_t group, scale_dtype;
    int32_t Kc, Nout;
    int64_t n_rows;                       // dense: M
    const int32_t* offsets;               // grouped: [E+1] row offsets (expert order); NULL = dense
    const int32_t* tile_offsets;          // grouped: [E+1] prefix of ceil(count/BM)
    int32_t num_experts;
    const bf16_t* su;                     // [rows, r_pad] or NULL
    const bf16_t* lora_right;             // [E][Nout][r_pad] or NULL
    int32_t r_pad;
    const bf16_t* bias;                   // [Nout] or NULL
};

// ------------------------------------------------------------------ W tile loaders
// Each loader fetches the packed bytes of the (n0, k0) tile into registers
// (load) and later decodes + writes them to Bs[n][kc] (store).

template <int FMT>
__device__ __forceinline__ void decode16_4bit(const u32x2 w, float s, float gs, float* v) {
    if (FMT == XQ_FMT_NVFP4) s = s * gs;
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = val4<FMT>((w[i >> 3] >> (4 * (i & 7))) & 0xfu, s);
}

__device__ __forceinline__ void lds_store_run16(bf16_t* dst, const float* v) {
    u32x4* o = (u32x4*)dst;
    o[0] = u32x4{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
    o[1] = u32x4{pack_bf16x2(v[8], v[9]), pack_bf16x2(v[10], v[11]), pack_bf16x2(v[12], v[13]), pack_bf16x2(v[14], v[15])};
}

// ---- block fp8 ----
template <bool CONTRACT_COLS>
struct LoaderFp8 {
    u32x4 raw[2];
    float s;
    __device__ __forceinline__ void load(const TileArgs& g, const uint8_t* pk, const uint8_t* sc, float, int n0, int k0, int tid) {
        const int scols = (g.wcols + 127) >> 7;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            int u = tid + p * 256;
            int row, col;
            if (CONTRACT_COLS) { row = n0 + (u >> 2); col = k0 + (u & 3) * 16; row = min(row, g.wrows - 1); }
            else { row = k0 + (u & 63); col = n0 + (u >> 6) * 16; col = min(col, g.wcols - 16); }
            raw[p] = *(const u32x4*)(pk + (int64_t)row * g.wcols + col);
        }
        int br = CONTRACT_COLS ? (n0 >> 7) : (k0 >> 7), bc = CONTRACT_COLS ? (k0 >> 7) : (n0 >> 7);
        s = ((const float*)sc)[br * scols + bc];
    }
    __device__ __forceinline__ void store(bf16_t* Bs, int tid) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            int u = tid + p * 256;
            float v[16];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f32x2 lo = e4m3x2_to_f32(raw[p][i], false), hi = e4m3x2_to_f32(raw[p][i], true);
                v[4 * i] = lo[0] * s; v[4 * i + 1] = lo[1] * s; v[4 * i + 2] = hi[0] * s; v[4 * i + 3] = hi[1] * s;
            }
            if (CONTRACT_COLS) {
                lds_store_run16(Bs + (u >> 2) * LDS_PITCH + (u & 3) * 16, v);
            } else {
                int kc = u & 63, nb = (u >> 6) * 16;
#pragma unroll
                for (int j = 0; j < 16; ++j) Bs[(nb + j) * LDS_PITCH + kc] = to_bf16(v[j]);
            }
        }
    }
};

// ---- 4-bit, FLAT storage (pairs and groups along W cols) ----
template <int FMT, bool CONTRACT_COLS>
struct Loader4Flat {
    u32x2 raw[2];
    float s[2];
    float gs;
    __device__ __forceinline__ void load(const TileArgs& g, const uint8_t* pk, const uint8_t* sc, float gscale, int n0, int k0, int tid) {
        gs = gscale;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            int u = tid + p * 256;
            int row, col;
            if (CONTRACT_COLS) { row = n0 + (u >> 2); col = k0 + (u & 3) * 16; row = min(row, g.wrows - 1); }
            else { row = k0 + (u & 63); col = n0 + (u >> 6) * 16; col = min(col, g.wcols - 16); }
            int64_t e = (int64_t)row * g.wcols + col;
            raw[p] = *(const u32x2*)(pk + (e >> 1));
            s[p] = load_scale(sc, e / g.group, g.scale_dtype);
        }
    }
    __device__ __forceinline__ void store(bf16_t* Bs, int tid) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            int u = tid + p * 256;
            float v[16];
            decode16_4bit<FMT>(raw[p], s[p], gs, v);
            if (CONTRACT_COLS) {
                lds_store_run16(Bs + (u >> 2) * LDS_PITCH + (u & 3) * 16, v);
            } else {
                int kc = u & 63, nb = (u >> 6) * 16;
#pragma unroll
                for (int j = 0; j < 16; ++j) Bs[(nb + j) * LDS_PITCH + kc] = to_bf16(v[j]);
            }
        }
    }
};

// ---- 4-bit, GKN storage (pairs and groups along W rows) ----
// requires group % 2 == 0 (always) -- the two rows of a byte share a scale.
template <int FMT, bool CONTRACT_COLS>
struct Loader4Gkn {
    u32x4 raw;
    float s[16];
    float gs;
    __device__ __forceinline__ void load(const TileArgs& g, const uint8_t* pk, const uint8_t* sc, float gscale, int n0, int k0, int tid) {
        gs = gscale;
        int r2, col;  // packed row, first col
        if (CONTRACT_COLS) { r2 = (n0 >> 1) + (tid >> 2); col = k0 + (tid & 3) * 16; r2 = min(r2, (g.wrows >> 1) - 1); }
        else { r2 = (k0 >> 1) + (tid & 31); col = n0 + (tid >> 5) * 16; col = min(col, g.wcols - 16); }
        raw = *(const u32x4*)(pk + (int64_t)r2 * g.wcols + col);
        int64_t sbase = (int64_t)((2 * r2) / g.group) * g.wcols + col;
#pragma unroll
        for (int i = 0; i < 16; ++i) s[i] = load_scale(sc, sbase + i, g.scale_dtype);
    }
    __device__ __forceinline__ void store(bf16_t* Bs, int tid) {
        float ve[16], vo[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            uint32_t b = (raw[i >> 2] >> (8 * (i & 3))) & 0xffu;
            float sc = s[i];
            if (FMT == XQ_FMT_NVFP4) sc = sc * gs;
            ve[i] = val4<FMT>(b & 0xfu, sc);
            vo[i] = val4<FMT>(b >> 4, sc);
        }
        if (CONTRACT_COLS) {
            int n = 2 * (tid >> 2), kc = (tid & 3) * 16;
            lds_store_run16(Bs + n * LDS_PITCH + kc, ve);
            lds_store_run16(Bs + (n + 1) * LDS_PITCH + kc, vo);
        } else {
            int kc = 2 * (tid & 31), nb = (tid >> 5) * 16;
#pragma unroll
            for (int j = 0; j < 16; ++j) *(uint32_t*)(Bs + (nb + j) * LDS_PITCH + kc) = pack_bf16x2(ve[j], vo[j]);
        }
    }
};

template <int FMT, int LAYOUT, bool CC> struct LoaderSel;
template <int LAYOUT, bool CC> struct LoaderSel<XQ_FMT_FP8, LAYOUT, CC> { using type = LoaderFp8<CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_INT4, XQ_LAYOUT_FLAT, CC> { using type = Loader4Flat<XQ_FMT_INT4, CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_NVFP4, XQ_LAYOUT_FLAT, CC> { using type = Loader4Flat<XQ_FMT_NVFP4, CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_INT4, XQ_LAYOUT_GKN, CC> { using type = Loader4Gkn<XQ_FMT_INT4, CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_NVFP4, XQ_LAYOUT_GKN, CC> { using type = Loader4Gkn<XQ_FMT_NVFP4, CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_NF4, XQ_LAYOUT_FLAT, CC> { using type = Loader4Flat<XQ_FMT_NF4, CC>; };
template <bool CC> struct LoaderSel<XQ_FMT_NF4, XQ_LAYOUT_GKN, CC> { using type = Loader4Gkn<XQ_FMT_NF4, CC>; };

// ------------------------------------------------------------------ the kernel
template <int FMT, int LAYOUT, bool CONTRACT_COLS>
__global__ void __launch_bounds__(256) gemm_tile_kernel(TileArgs g) {
    __shared__ __attribute__((aligned(16))) bf16_t As[BM * LDS_PITCH];
    __shared__ __attribute__((aligned(16))) bf16_t Bs[BN * LDS_PITCH];
    __shared__ int sh_info[3];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- which rows / which expert
    int e = 0;
    int64_t row0, row_end;
    if (g.offsets) {
        if (tid == 0) {
            int t = blockIdx.x, lo = 0, hi = g.num_experts;  // find e: tile_offsets[e] <= t < tile_offsets[e+1]
            if (t >= g.tile_offsets[g.num_experts]) { sh_info[0] = -1; }
            else {
                while (hi - lo > 1) { int mid = (lo + hi) >> 1; if (g.tile_offsets[mid] <= t) lo = mid; else hi = mid; }
                sh_info[0] = lo;
                sh_info[1] = g.offsets[lo] + (t - g.tile_offsets[lo]) * BM;
                sh_info[2] = g.offsets[lo + 1];
            }
        }
        __syncthreads();
        e = sh_info[0];
        if (e < 0) return;
        row0 = sh_info[1];
        row_end = sh_info[2];
    } else {
        row0 = (int64_t)blockIdx.x * BM;
        row_end = g.n_rows;
        if (row0 >= row_end) return;
    }
    const int n0 = blockIdx.y * BN;
    const uint8_t* pk = g.packed + (int64_t)e * g.packed_stride;
    const uint8_t* sc = g.scales + (int64_t)e * g.scale_stride;
    const float gscale = (FMT == XQ_FMT_NVFP4) ? g.global_scale[e] : 1.0f;

    typename LoaderSel<FMT, LAYOUT, CONTRACT_COLS>::type wl;
    u32x4 areg[4];

    auto load_a = [&](int k0) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            int64_t r = row0 + p * 32 + (tid >> 3);
            r = r < row_end ? r : row_end - 1;
            areg[p] = *(const u32x4*)(g.A + r * g.lda + k0 + (tid & 7) * 8);
        }
    };
    auto store_a = [&]() {
#pragma unroll
        for (int p = 0; p < 4; ++p) *(u32x4*)(As + (p * 32 + (tid >> 3)) * LDS_PITCH + (tid & 7) * 8) = areg[p];
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;

    auto mma_steps = [&](int nsteps) {
        const int fr = lane & 31, fk = (lane >> 5) * 8;
        for (int ks = 0; ks < nsteps; ++ks) {
            bf16x8 a[2], b[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                a[i] = *(const bf16x8*)(As + (wm * 64 + i * 32 + fr) * LDS_PITCH + ks * 16 + fk);
                b[i] = *(const bf16x8*)(Bs + (wn * 64 + i * 32 + fr) * LDS_PITCH + ks * 16 + fk);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }
    };

    const int nk = g.Kc / BK;
    load_a(0);
    wl.load(g, pk, sc, gscale, n0, 0, tid);
    store_a();
    wl.store(Bs, tid);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
        const bool more = kt + 1 < nk;
        if (more) {
            load_a((kt + 1) * BK);
            wl.load(g, pk, sc, gscale, n0, (kt + 1) * BK, tid);
        }
        mma_steps(BK / 16);
        __syncthreads();
        if (more) {
            store_a();
            wl.store(Bs, tid);
        }
        __syncthreads();
    }

    // ---- low-rank side term: one more K-step of width r_pad
    if (g.r_pad > 0) {
        const int rp = g.r_pad;  // multiple of 16, <= 64
        // As <- su[rows, rp], Bs <- lora_right[e][n, rp]; both zero beyond rp are never read
        for (int idx = tid; idx < BM * (rp / 8); idx += 256) {
            int r = idx / (rp / 8), c = (idx % (rp / 8)) * 8;
            int64_t row = row0 + r;
            row = row < row_end ? row : row_end - 1;
            *(u32x4*)(As + r * LDS_PITCH + c) = *(const u32x4*)(g.su + row * rp + c);
            int n = n0 + r;
            n = n < g.Nout ? n : g.Nout - 1;
            *(u32x4*)(Bs + r * LDS_PITCH + c) = *(const u32x4*)(g.lora_right + ((int64_t)e * g.Nout + n) * rp + c);
        }
        __syncthreads();
        mma_steps(rp / 16);
    }

    // ---- epilogue: fp32 -> bf16, masked rows/cols
    const int col_l = lane & 31, rgrp = (lane >> 5) * 4;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        int n = n0 + wn * 64 + j * 32 + col_l;
        if (n >= g.Nout) continue;
        float bv = g.bias ? bf16_to_f32(g.bias[n]) : 0.0f;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                int64_t row = row0 + wm * 64 + i * 32 + (q & 3) + rgrp + 8 * (q >> 2);
                if (row < row_end) g.C[row * g.ldc + n] = to_bf16(acc[i][j][q] + bv);
            }
        }
    }
}

}  // namespace xq
