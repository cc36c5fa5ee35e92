// Low-rank helper kernels (see xq_lora.h).  bf16 MFMA, fp32 accumulate.
#include "xq_lora.h"
#include <atomic>

namespace xq {

// ------------------------------------------------------------------ zero fill
__global__ void __launch_bounds__(256) zero_fill_kernel(u32x4* p, int64_t n16, uint8_t* tail, int tail_bytes) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n16) p[i] = u32x4{0, 0, 0, 0};
    if (i == 0)
        for (int t = 0; t < tail_bytes; ++t) tail[t] = 0;
}

int launch_zero_fill(void* p, int64_t bytes, hipStream_t stream) {
    if (bytes <= 0) return XQ_OK;
    XQ_REQUIRE(xq_aligned(p, 16), "zero_fill: pointer not 16-byte aligned");
    int64_t n16 = bytes / 16;
    int tail = (int)(bytes - n16 * 16);
    int64_t blocks = xq_cdiv(n16 > 0 ? n16 : 1, 256);
    zero_fill_kernel<<<dim3((unsigned)blocks), 256, 0, stream>>>((u32x4*)p, n16, (uint8_t*)p + n16 * 16, tail);
    XQ_CHECK_LAUNCH("zero_fill");
    return XQ_OK;
}

// ------------------------------------------------------------------ factor prep
__global__ void __launch_bounds__(256) factor_prep_kernel(const void* in, int in_f32, int64_t R_in, int64_t C_in,
                                                          int transpose, bf16_t* out, int64_t R_out, int64_t C_out,
                                                          int64_t total) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total) return;
    int64_t per = R_out * C_out;
    int64_t e = t / per, rem = t - e * per;
    int64_t i = rem / C_out, j = rem - i * C_out;
    int64_t si = transpose ? j : i, sj = transpose ? i : j;
    float v = 0.0f;
    if (si < R_in && sj < C_in) {
        int64_t idx = e * R_in * C_in + si * C_in + sj;
        v = in_f32 ? ((const float*)in)[idx] : bf16_to_f32(((const bf16_t*)in)[idx]);
    }
    out[t] = to_bf16(v);
}

int launch_factor_prep(const void* in, int in_dtype, int64_t R_in, int64_t C_in, bool transpose, bf16_t* out,
                       int64_t R_out, int64_t C_out, int64_t num_experts, hipStream_t stream) {
    int64_t total = num_experts * R_out * C_out;
    if (total == 0) return XQ_OK;
    factor_prep_kernel<<<dim3((unsigned)xq_cdiv(total, 256)), 256, 0, stream>>>(in, in_dtype == XQ_DT_F32, R_in, C_in,
                                                                                transpose, out, R_out, C_out, total);
    XQ_CHECK_LAUNCH("factor_prep");
    return XQ_OK;
}

// Two or three dense factor conversions in one launch (blockIdx.y = job): the linear entry points prepare both
// factors of a call together, which matters where a step is a dozen short launches.
__global__ void __launch_bounds__(256) factor_prep_multi_kernel(FactorPrepJobs j) {
    const int k = blockIdx.y;
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t R_out = j.R_out[k], C_out = j.C_out[k], R_in = j.R_in[k], C_in = j.C_in[k];
    if (t >= R_out * C_out) return;
    const int64_t i = t / C_out, c = t - i * C_out;
    const int64_t si = j.transpose[k] ? c : i, sj = j.transpose[k] ? i : c;
    float v = 0.0f;
    if (si < R_in && sj < C_in) {
        const int64_t idx = si * C_in + sj;
        v = j.in_f32 ? ((const float*)j.in[k])[idx] : bf16_to_f32(((const bf16_t*)j.in[k])[idx]);
    }
    j.out[k][t] = to_bf16(v);
}

int launch_factor_prep_multi(const FactorPrepJobs& j, hipStream_t stream) {
    int64_t most = 0;
    for (int k = 0; k < j.n; ++k) most = j.R_out[k] * j.C_out[k] > most ? j.R_out[k] * j.C_out[k] : most;
    if (j.n == 0 || most == 0) return XQ_OK;
    factor_prep_multi_kernel<<<dim3((unsigned)xq_cdiv(most, 256), (unsigned)j.n), 256, 0, stream>>>(j);
    XQ_CHECK_LAUNCH("factor_prep_multi");
    return XQ_OK;
}

// A block converts one tile of a destination panel through LDS -- 16 x 256 (rows x columns) of a wide panel, 256 x 16
// of a tall one -- so that both the source and the destination are touched in whole row pieces whichever way the job
// transposes: e.g. a transposing job into a wide panel reads 256 source rows of 16 entries (one contiguous run when
// the factor is 16 wide) and writes 16 destination rows of 512 bytes.  (Element by element, the transposing jobs of
// an expert bank read 4 bytes of every 64-byte row piece per instruction: 61 us for the panels of 128 experts.)
// Every load is unconditional (indices past the source clamped onto it, the value replaced by zero afterwards): with a
// branch around them the compiler waits for each load before it issues the next, sixteen round trips per tile.
constexpr int PP_S = 16, PP_L = 256;
template <bool F32>
__global__ void __launch_bounds__(256) panel_prep_kernel(PanelJobs j) {
    __shared__ float tile[PP_L][PP_S + 1];      // [index along the tile's long side][along its short side]
    const int k = blockIdx.y, tid = threadIdx.x;
    const int64_t R_in = j.R_in[k], C_in = j.C_in[k], C_out = j.C_out[k], R_out = j.R_out[k], pitch = j.pitch[k];
    const bool tr = j.transpose[k] != 0, shared = j.n_src[k] == 1;
    const void* in = j.in[k];
    bf16_t* out = j.out[k];
    const int64_t e_stride = j.e_stride[k];
    const bool wide = C_out >= R_out;           // the long side runs along the destination's columns
    const int64_t TRW = wide ? PP_S : PP_L, TCW = wide ? PP_L : PP_S;
    const int64_t tiles_r = (R_out + TRW - 1) / TRW, tiles_c = (C_out + TCW - 1) / TCW;
    const int64_t total = tiles_r * tiles_c * j.n_out[k];
    const bool load_long_first = wide != tr;    // consecutive threads walk along the source's rows
    for (int64_t t = blockIdx.x; t < total; t += gridDim.x) {
        const int64_t e = t / (tiles_r * tiles_c), rem = t - e * (tiles_r * tiles_c);
        const int64_t i0 = (rem / tiles_c) * TRW, c0 = (rem % tiles_c) * TCW;
        const int64_t base = (shared ? 0 : e) * R_in * C_in;
        float val[PP_S];
        uint32_t keep = 0xffffu;
#pragma unroll
        for (int u = 0; u < PP_S; ++u) {
            const int idx = u * 256 + tid;
            const int l = load_long_first ? idx % PP_L : idx / PP_S, sh = load_long_first ? idx / PP_L : idx % PP_S;
            const int64_t i = i0 + (wide ? sh : l), c = c0 + (wide ? l : sh);
            const int64_t si = tr ? c : i, sj = tr ? i : c;
            const int64_t src = base + (si < R_in ? si : R_in - 1) * C_in + (sj < C_in ? sj : C_in - 1);
            val[u] = F32 ? ((const float*)in)[src] : bf16_to_f32(((const bf16_t*)in)[src]);
            if (!(si < R_in && sj < C_in)) keep &= ~(1u << u);
        }
#pragma unroll
        for (int u = 0; u < PP_S; ++u) {
            const int idx = u * 256 + tid;
            const int l = load_long_first ? idx % PP_L : idx / PP_S, sh = load_long_first ? idx / PP_L : idx % PP_S;
            tile[l][sh] = (keep >> u) & 1u ? val[u] : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < PP_S; ++u) {
            const int idx = u * 256 + tid;      // consecutive threads walk along the destination's rows
            const int l = wide ? idx % PP_L : idx / PP_S, sh = wide ? idx / PP_L : idx % PP_S;
            const int64_t i = i0 + (wide ? sh : l), c = c0 + (wide ? l : sh);
            if (i < R_out && c < C_out) out[e * e_stride + i * pitch + c] = to_bf16(tile[l][sh]);
        }
        __syncthreads();
    }
}

int launch_panel_prep(const PanelJobs& j, hipStream_t stream) {
    int64_t most = 0;
    for (int k = 0; k < j.n; ++k) {
        const bool wide = j.C_out[k] >= j.R_out[k];
        const int64_t t = xq_cdiv(j.R_out[k], wide ? PP_S : PP_L) * xq_cdiv(j.C_out[k], wide ? PP_L : PP_S) * j.n_out[k];
        most = t > most ? t : most;
    }
    if (j.n == 0 || most == 0) return XQ_OK;
    if (most > 16384) most = 16384;
    if (j.in_f32) panel_prep_kernel<true><<<dim3((unsigned)most, (unsigned)j.n), 256, 0, stream>>>(j);
    else panel_prep_kernel<false><<<dim3((unsigned)most, (unsigned)j.n), 256, 0, stream>>>(j);
    XQ_CHECK_LAUNCH("panel_prep");
    return XQ_OK;
}

// ------------------------------------------------------------------ small_nt
struct SmallNtArgs {
    const bf16_t* In;
    int64_t ld_in;
    int64_t n_rows;
    int64_t Kc;
    const bf16_t* F;
    int64_t f_stride;  // elements per expert (0 = shared)
    int r_pad;
    float scale;
    bf16_t* T;
    int64_t ld_t;      // row pitch of T (and T2) in elements
    bf16_t* T2;        // optional: result columns from `split` on go to T2 (as its columns 0 ..) instead of T
    int split;
    const int32_t* offsets;
    const int32_t* tile_offsets;
    int32_t num_experts;
    // grouped, optional: row i of the product is made from row row_map[i] of In (rows gathered from a compact matrix),
    // and the gathered rows are also written to copy_out (row pitch ld_copy) -- the row permutation of a routed
    // problem rides on the pass that reads the rows first instead of being a pass of its own
    const int32_t* row_map;
    bf16_t* copy_out;
    int64_t ld_copy;
};

// TR rows per block: 32 (dense; the 4 waves split K) or 128 (grouped; one wave per 32 rows).  FJ = rows of F in
// use / 4 (4, 8, 12 or 16).
// Both operands are fetched with coalesced 16-byte loads (16 lanes per 256-byte row piece, 4 rows
// per instruction) and reach the MFMA operand layout through wave-private LDS tiles of 128 k per
// row (row pitch 272 B: the 16 lanes of a b128 read phase hit distinct banks); per-lane row-strided
// loads would touch 64 cache lines per instruction and leave the kernel address-unit bound.
// A wave keeps two 128-k chunks of its activation rows in flight (the factor chunk, which comes from L2, one):
// every load is unconditional -- rows past the segment and columns past the wave's K range are clamped onto
// valid ones and their values never used -- so the waits count exactly and the loads of chunk k+2 stay in
// flight while chunk k is multiplied.
constexpr int SN_P = 136;   // LDS row pitch in bf16 elements
template <int TR, int FJ, bool GATHER = false>
__global__ void __launch_bounds__(256) small_nt_kernel(SmallNtArgs g) {
    constexpr int NT = (FJ + 7) / 8;
    constexpr int RG = TR / 32, KS = 4 / RG;
    constexpr int WTILE = (32 + NT * 32) * SN_P;   // bf16 elements per wave: In tile + F tile
    extern __shared__ __attribute__((aligned(16))) bf16_t sn_lds[];
    __shared__ int sh_info[3];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rg = wave % RG, ks = wave / RG;

    int e = 0;
    int64_t row0, row_end;
    if (g.offsets) {
        // the expert whose tile range holds this block's tile: one look per thread, all loads in flight together
        // (a binary search by one thread is a chain of dependent memory round trips)
        if (tid == 0) sh_info[0] = -1;
        __syncthreads();
        const int t = blockIdx.x;
        for (int x = tid; x < g.num_experts; x += blockDim.x) {
            const int lo = g.tile_offsets[x], hi = g.tile_offsets[x + 1];
            const int o0 = g.offsets[x], o1 = g.offsets[x + 1];
            if (lo <= t && t < hi) {
                sh_info[0] = x;
                sh_info[1] = o0 + (t - lo) * TR;
                sh_info[2] = o1;
            }
        }
        __syncthreads();
        e = sh_info[0];
        if (e < 0) return;
        row0 = sh_info[1];
        row_end = sh_info[2];
    } else {
        row0 = (int64_t)blockIdx.x * TR;
        row_end = g.n_rows;
        if (row0 >= row_end) return;
    }
    const bf16_t* F = g.F + (int64_t)e * g.f_stride;
    bf16_t* xs = sn_lds + wave * WTILE;          // [32][SN_P]
    bf16_t* fs = xs + 32 * SN_P;                 // [NT*32][SN_P]
    const int fr = lane & 31, fk = (lane >> 5) * 8;
    const int crow = lane >> 4, cpiece = (lane & 15) * 8;   // coalesced fetch: row within a group of 4, k offset
    const int64_t wrow0 = row0 + rg * 32;
    const int frows = g.r_pad;                   // rows of F in use (= 4 * FJ)

    f32x16 acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[n][q] = 0.0f;

    const int64_t kspan = g.Kc / KS;  // multiple of 16
    const int64_t kbeg = ks * kspan, kend = kbeg + kspan;
    const bf16_t* xp[8];
    int32_t orow[GATHER ? 8 : 1];                // GATHER: the rows of copy_out this lane's pieces belong to
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        int64_t r = wrow0 + j * 4 + crow;
        r = r < row_end ? r : row_end - 1;       // wrow0 may lie past a short segment's end: still a valid row
        r = r < 0 ? 0 : r;
        if constexpr (GATHER) {
            orow[j] = (int32_t)r;
            xp[j] = g.In + (int64_t)g.row_map[r] * g.ld_in;
        } else {
            xp[j] = g.In + r * g.ld_in;
        }
    }
    u32x4 xr[2][8], fq[FJ];
    auto fetch_x = [&](u32x4* dst, int64_t k) {  // chunk [k, k+128); pieces past kend come from the range's last piece
        int64_t kc = k + cpiece;
        kc = kc < kend ? kc : kend - 8;
#pragma unroll
        for (int j = 0; j < 8; ++j) dst[j] = *(const u32x4*)(xp[j] + kc);
    };
    auto fetch_f = [&](int64_t k) {
        int64_t kc = k + cpiece;
        kc = kc < kend ? kc : kend - 8;
#pragma unroll
        for (int j = 0; j < FJ; ++j) fq[j] = *(const u32x4*)(F + (int64_t)(j * 4 + crow) * g.Kc + kc);
    };
    auto chunk = [&](u32x4* cur, int64_t k) {    // multiply chunk k out of `cur`; refill it with chunk k + 256
        // LDS operations of one wave execute in order: the previous chunk's fragment reads are ahead of these writes
#pragma unroll
        for (int j = 0; j < 8; ++j) *(u32x4*)(xs + (j * 4 + crow) * SN_P + cpiece) = cur[j];
#pragma unroll
        for (int j = 0; j < FJ; ++j) *(u32x4*)(fs + (j * 4 + crow) * SN_P + cpiece) = fq[j];
        if constexpr (GATHER) {
            // (rows and pieces that were clamped onto valid ones are written again with the same bytes)
            int64_t kc = k + cpiece;
            kc = kc < kend ? kc : kend - 8;
            if (g.copy_out && k < kend) {
#pragma unroll
                for (int j = 0; j < 8; ++j) *(u32x4*)(g.copy_out + (int64_t)orow[j] * g.ld_copy + kc) = cur[j];
            }
        }
        fetch_f(k + 128);
        fetch_x(cur, k + 256);
        const int64_t left = kend - k;           // <= 0 for the idle second half of the last pair
        const int nsteps = (int)((left < 128 ? (left < 0 ? 0 : left) : 128) >> 4);
#pragma unroll
        for (int st = 0; st < 8; ++st) {
            if (st < nsteps) {                   // uniform
                const bf16x8 a = *(const bf16x8*)(xs + fr * SN_P + st * 16 + fk);
#pragma unroll
                for (int n = 0; n < NT; ++n) {
                    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
                    const bf16x8 b = (n * 32 + fr < frows) ? *(const bf16x8*)(fs + (n * 32 + fr) * SN_P + st * 16 + fk) : zero8;
                    acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[n], 0, 0, 0);
                }
            }
        }
    };
    fetch_x(xr[0], kbeg);
    fetch_f(kbeg);
    fetch_x(xr[1], kbeg + 128);
    for (int64_t k = kbeg; k < kend; k += 256) {
        chunk(xr[0], k);
        chunk(xr[1], k + 128);
    }

    if (KS > 1) {
        float* red = (float*)sn_lds;   // [(KS-1)][NT][16][64] floats, over the (now dead) tiles
        __syncthreads();
        if (ks > 0) {
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
                for (int q = 0; q < 16; ++q) red[(((ks - 1) * NT + n) * 16 + q) * 64 + lane] = acc[n][q];
        }
        __syncthreads();
        if (ks > 0) return;
#pragma unroll
        for (int s = 1; s < KS; ++s)
#pragma unroll
            for (int n = 0; n < NT; ++n)
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[n][q] += red[(((s - 1) * NT + n) * 16 + q) * 64 + lane];
    }
    const int rgrp = (lane >> 5) * 4;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        int j = n * 32 + fr;
        if (j >= g.r_pad) continue;
        bf16_t* dst = g.T;
        int jj = j;
        if (g.T2 && j >= g.split) { dst = g.T2; jj = j - g.split; }
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            int64_t row = row0 + rg * 32 + (q & 3) + rgrp + 8 * (q >> 2);
            if (row < row_end) dst[row * g.ld_t + jj] = to_bf16(acc[n][q] * g.scale);
        }
    }
}

template <int TR, int FJ, bool GATHER = false>
static int launch_small_nt_one(const SmallNtArgs& g, unsigned blocks, hipStream_t stream) {
    constexpr int NT = (FJ + 7) / 8;
    constexpr size_t lds = (size_t)4 * (32 + NT * 32) * SN_P * 2;
    static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)small_nt_kernel<TR, FJ, GATHER>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            xq_set_error("small_nt: cannot raise the dynamic LDS limit: %s", hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    small_nt_kernel<TR, FJ, GATHER><<<dim3(blocks), 256, lds, stream>>>(g);
    return XQ_OK;
}

template <int TR, bool GATHER = false>
static int launch_small_nt_rows(const SmallNtArgs& g, unsigned blocks, hipStream_t stream) {
    switch (g.r_pad) {
        case 16: return launch_small_nt_one<TR, 4, GATHER>(g, blocks, stream);
        case 32: return launch_small_nt_one<TR, 8, GATHER>(g, blocks, stream);
        case 48: return launch_small_nt_one<TR, 12, GATHER>(g, blocks, stream);
        default: return launch_small_nt_one<TR, 16, GATHER>(g, blocks, stream);
    }
}

int launch_small_nt(const bf16_t* In, int64_t ld_in, int64_t n_rows, int64_t Kc, const bf16_t* F, int r_pad,
                    float scale, bf16_t* T, const int32_t* offsets, const int32_t* tile_offsets,
                    int32_t num_experts, bool shared_f, hipStream_t stream, int64_t ld_t, bf16_t* T2, int split,
                    const int32_t* row_map, bf16_t* copy_out, int64_t ld_copy) {
    if (ld_t <= 0) ld_t = r_pad;
    if (T2) XQ_REQUIRE(split > 0 && split < r_pad && ld_t >= split && ld_t >= r_pad - split, "small_nt: bad split of the result columns");
    else XQ_REQUIRE(ld_t >= r_pad, "small_nt: output pitch %lld below r_pad %d", (long long)ld_t, r_pad);
    XQ_REQUIRE(r_pad > 0 && r_pad <= 64 && r_pad % 16 == 0, "small_nt: r_pad must be 16/32/48/64, got %d", r_pad);
    XQ_REQUIRE(Kc % 64 == 0, "small_nt: contraction length %lld must be a multiple of 64", (long long)Kc);
    XQ_REQUIRE(ld_in % 8 == 0 && xq_aligned(In, 16) && xq_aligned(F, 16), "small_nt: operands must be 16-byte aligned");
    if (n_rows == 0) return XQ_OK;
    XQ_REQUIRE(!row_map || (offsets && (!copy_out || (ld_copy % 8 == 0 && ld_copy >= Kc && xq_aligned(copy_out, 16)))),
               "small_nt: gathered rows need the grouped form, and a copy of them a 16-byte aligned copy_out");
    SmallNtArgs g{In, ld_in, n_rows, Kc, F, shared_f ? 0 : (int64_t)r_pad * Kc, r_pad, scale, T, ld_t, T2, split, offsets,
                  tile_offsets, num_experts, row_map, copy_out, ld_copy};
    int rc;
    if (offsets && row_map) {
        rc = launch_small_nt_rows<128, true>(g, (unsigned)(xq_cdiv(n_rows, 128) + num_experts), stream);
    } else if (offsets) {
        rc = launch_small_nt_rows<128>(g, (unsigned)(xq_cdiv(n_rows, 128) + num_experts), stream);
    } else {
        g.f_stride = 0;
        rc = launch_small_nt_rows<32>(g, (unsigned)xq_cdiv(n_rows, 32), stream);
    }
    if (rc) return rc;
    XQ_CHECK_LAUNCH("small_nt");
    return XQ_OK;
}

// ------------------------------------------------------------------ SwiGLU backward + its two low-rank products
// One pass over (gate, up, dh): writes dgate | dup (the elementwise kernel's arithmetic, ops/moe/lora.py:855-917 with no
// routing weight) and forms Tg = s * dgate . Fg^T and Tu = s * dup . Fu^T from the values on their way out -- the two
// products no longer read dgate | dup back.  Dense rows; organisation and summation order of small_nt_kernel<32, FJ>
// (32 rows per block, the four waves split the columns, 128 columns at a time through wave-private LDS tiles), so Tg
// and Tu are the bits the two small_nt launches produce.
struct SiluNtArgs {
    const bf16_t* gate;
    const bf16_t* up;
    int64_t ld_gu;
    const bf16_t* dh;
    int64_t ld_dh;
    bf16_t* dgate;
    bf16_t* dup;
    int64_t ld_out;
    int64_t n_rows, Kc;        // rows; columns of gate / up / dh (the contraction length of the two products)
    const bf16_t* Fg;          // [r_pad][Kc]
    const bf16_t* Fu;
    int r_pad;
    float scale;
    bf16_t* Tg;                // [n_rows][ld_t]
    bf16_t* Tu;
    int64_t ld_t;
    // routed rows (GROUPED): rows in expert order, a factor pair per expert (stride 0: shared), the routing weight of a row
    // applied as the elementwise kernel applies it, and its gradient
    const int32_t* offsets;
    const int32_t* tile_offsets;
    int32_t num_experts;
    int64_t fg_stride, fu_stride;
    const float* row_w;
    float* d_row_w;
    float limit;               // SwiGLU limit on the gate pre-activation (<= 0: none)
};

// GROUPED: routed rows in expert order, organisation of small_nt_kernel<128, FJ> (a block = a 128-row tile of one expert, a
// wave = 32 rows over all columns, the expert's own factor pair), the routing weight applied and its gradient formed as
// the elementwise kernel does (the sum over a row runs in another order here: 16 lanes' partial sums, then a butterfly).
// FWD: the forward pass in the same organisation -- h = bf16(bf16(silu(gate)) * up) (routed: then rounded and times the row's
// weight), the elementwise forward kernel's arithmetic, written through `dgate`, and Tg = scale * h . Fg^T from the values
// on their way out (dh, dup, Fu, Tu, d_row_w unused).
template <int FJ, bool GROUPED, bool FWD = false>
__global__ void __launch_bounds__(256, 2) silu_bwd_nt_kernel(SiluNtArgs g) {
    static_assert(FJ <= 8, "one MFMA column tile per product");
    // 64 columns at a time (where small_nt_kernel takes 128: the same MFMA steps in the same order): three operands' pieces
    // are 12 KB per wave in flight, and two blocks share a compute unit
    constexpr int CW = 64, P = CW + 8;           // columns of a chunk; LDS row pitch (144 B: the 16 lanes of a read phase hit distinct banks)
    constexpr int NL = 32 * CW / 512;            // 16-byte loads per lane and operand chunk (a load instruction covers 512 / CW rows)
    constexpr int RPI = 512 / CW;                // rows per load instruction
    constexpr int FL = (FJ * 4 + RPI - 1) / RPI; // loads per lane of a factor chunk (FJ * 4 rows)
    constexpr int WTILE = (32 + 32) * P;         // bf16 elements per wave: value tile + factor tile
    extern __shared__ __attribute__((aligned(16))) bf16_t sn_lds[];
    __shared__ int sh_info[3];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    int e = 0;
    int64_t row0, row_end;
    if constexpr (GROUPED) {
        // the expert whose tile range holds this block's tile: one look per thread, all loads in flight together
        if (tid == 0) sh_info[0] = -1;
        __syncthreads();
        const int t = blockIdx.x;
        for (int x = tid; x < g.num_experts; x += 256) {
            const int lo = g.tile_offsets[x], hi = g.tile_offsets[x + 1];
            const int o0 = g.offsets[x], o1 = g.offsets[x + 1];
            if (lo <= t && t < hi) {
                sh_info[0] = x;
                sh_info[1] = o0 + (t - lo) * 128;
                sh_info[2] = o1;
            }
        }
        __syncthreads();
        e = sh_info[0];
        if (e < 0) return;
        row0 = sh_info[1] + wave * 32;
        row_end = sh_info[2];
        if (row0 >= row_end) return;             // (no block barrier from here on in this form)
    } else {
        row0 = (int64_t)blockIdx.x * 32;
        row_end = g.n_rows;
        if (row0 >= row_end) return;
    }
    const bf16_t* Fg = g.Fg + (int64_t)e * g.fg_stride;
    const bf16_t* Fu = g.Fu + (int64_t)e * g.fu_stride;
    bf16_t* xs = sn_lds + wave * WTILE;          // [32][P]
    bf16_t* fs = xs + 32 * P;                    // [32][P]
    const int fr = lane & 31, fk = (lane >> 5) * 8;
    const int crow = lane / (CW / 8), cpiece = (lane % (CW / 8)) * 8;
    const int frows = g.r_pad;
    const int64_t kspan = GROUPED ? g.Kc : g.Kc / 4;        // multiple of 16
    const int64_t kbeg = GROUPED ? 0 : wave * kspan, kend = kbeg + kspan;
    const int64_t rbase = row0 + crow;           // this lane's rows: rbase + RPI j, clamped onto the last row
    auto row_of = [&](int j) { const int64_t r = rbase + j * RPI; return r < row_end ? r : row_end - 1; };
    float rw[GROUPED ? NL : 1], wsum[GROUPED ? NL : 1];
    if constexpr (GROUPED) {
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            rw[j] = g.row_w[row_of(j)];
            wsum[j] = 0.0f;
        }
    }
    u32x4 gq[NL], uq[NL], dq[NL], fq[FL];
    // every load is unconditional: rows past the end and pieces past the wave's columns are clamped onto valid ones
    auto fetch = [&](int64_t k) {
        int64_t kc = k + cpiece;
        kc = kc < kend ? kc : kend - 8;
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            const int64_t r = row_of(j);
            gq[j] = *(const u32x4*)(g.gate + r * g.ld_gu + kc);
            uq[j] = *(const u32x4*)(g.up + r * g.ld_gu + kc);
            if constexpr (!FWD) dq[j] = *(const u32x4*)(g.dh + r * g.ld_dh + kc);
        }
    };
    auto fetch_f = [&](const bf16_t* F, int64_t k) {
        int64_t kc = k + cpiece;
        kc = kc < kend ? kc : kend - 8;
#pragma unroll
        for (int j = 0; j < FL; ++j) fq[j] = *(const u32x4*)(F + (int64_t)(j * RPI + crow < FJ * 4 ? j * RPI + crow : FJ * 4 - 1) * g.Kc + kc);
    };
    auto stage_f = [&]() {
#pragma unroll
        for (int j = 0; j < FL; ++j)
            if (j * RPI + crow < 32) *(u32x4*)(fs + (j * RPI + crow) * P + cpiece) = fq[j];
    };
    f32x16 acc_g, acc_u;
#pragma unroll
    for (int q = 0; q < 16; ++q) acc_g[q] = acc_u[q] = 0.0f;
    auto multiply = [&](f32x16& acc, int nsteps) {
#pragma unroll
        for (int st = 0; st < CW / 16; ++st) {
            if (st < nsteps) {                   // uniform
                const bf16x8 a = *(const bf16x8*)(xs + fr * P + st * 16 + fk);
                const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
                const bf16x8 b = fr < frows ? *(const bf16x8*)(fs + fr * P + st * 16 + fk) : zero8;
                acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc, 0, 0, 0);
            }
        }
    };
    // The factor chunks (from L2) are requested ahead of the value chunks and go to the LDS tile as soon as the MFMAs that
    // read its previous contents are issued (LDS operations of one wave execute in order), so their registers are free
    // while a chunk's values are worked out.
    fetch_f(Fg, kbeg);
    fetch(kbeg);
    stage_f();
    if constexpr (FWD) {
        for (int64_t k = kbeg; k < kend; k += CW) {
            const int64_t kc = k + cpiece;
            const bool mine = kc < kend;
#pragma unroll
            for (int j = 0; j < NL; ++j) {
                u32x4 oh;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    float res[2];
#pragma unroll
                    for (int hlf = 0; hlf < 2; ++hlf) {
                        const float gv = swiglu_clamp(bf16_to_f32((bf16_t)(gq[j][i] >> (16 * hlf))), g.limit), uv = bf16_to_f32((bf16_t)(uq[j][i] >> (16 * hlf)));
                        const float a = round_bf16(gv * sigmoid_f32(gv));
                        float v = a * uv;
                        if constexpr (GROUPED) v = round_bf16(v) * rw[j];
                        res[hlf] = v;
                    }
                    oh[i] = pack_bf16x2(res[0], res[1]);
                }
                if (rbase + j * RPI < row_end && mine) *(u32x4*)(g.dgate + (rbase + j * RPI) * g.ld_out + kc) = oh;
                *(u32x4*)(xs + (j * RPI + crow) * P + cpiece) = oh;
            }
            fetch_f(Fg, k + CW);                // (past the last chunk: clamped, never used)
            fetch(k + CW);
            const int64_t left = kend - k;
            multiply(acc_g, (int)((left < CW ? left : CW) >> 4));
            stage_f();
        }
    } else
    for (int64_t k = kbeg; k < kend; k += CW) {
        const int64_t kc = k + cpiece;
        const bool mine = kc < kend;             // this lane's piece lies in the wave's columns
        fetch_f(Fu, k);
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            u32x4 og, ou;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                float rg[2], ru[2];
#pragma unroll
                for (int hlf = 0; hlf < 2; ++hlf) {
                    const float g_raw = bf16_to_f32((bf16_t)(gq[j][i] >> (16 * hlf))), uv = bf16_to_f32((bf16_t)(uq[j][i] >> (16 * hlf)));
                    const float gv = swiglu_clamp(g_raw, g.limit), open = swiglu_mask(g_raw, g.limit);
                    const float d = bf16_to_f32((bf16_t)(dq[j][i] >> (16 * hlf)));
                    const float sg = sigmoid_f32(gv);
                    const float a = round_bf16(gv * sg);
                    float dp = d;
                    if constexpr (GROUPED) {
                        dp = round_bf16(d * rw[j]);
                        if (mine) wsum[j] += d * round_bf16(a * uv);
                    }
                    rg[hlf] = round_bf16(dp * uv) * (sg * (1.0f + gv * (1.0f - sg))) * open;
                    ru[hlf] = a * dp;
                }
                og[i] = pack_bf16x2(rg[0], rg[1]);
                ou[i] = pack_bf16x2(ru[0], ru[1]);
            }
            if (rbase + j * RPI < row_end && mine) {
                const int64_t r = rbase + j * RPI;
                *(u32x4*)(g.dgate + r * g.ld_out + kc) = og;
                *(u32x4*)(g.dup + r * g.ld_out + kc) = ou;
            }
            *(u32x4*)(xs + (j * RPI + crow) * P + cpiece) = og;
            uq[j] = ou;                          // waits in registers for its turn in the tile
        }
        const int64_t left = kend - k;
        const int nsteps = (int)((left < CW ? left : CW) >> 4);
        multiply(acc_g, nsteps);
#pragma unroll
        for (int j = 0; j < NL; ++j) *(u32x4*)(xs + (j * RPI + crow) * P + cpiece) = uq[j];
        stage_f();                               // the up factor's chunk
        fetch_f(Fg, k + CW);                    // (past the last chunk: clamped, never used)
        fetch(k + CW);
        multiply(acc_u, nsteps);
        stage_f();                               // the gate factor's next chunk
    }

    const int rgrp = (lane >> 5) * 4;
    if constexpr (GROUPED) {
#pragma unroll
        for (int j = 0; j < NL; ++j) {
            float v = wsum[j];
#pragma unroll
            for (int o = 1; o < CW / 8; o <<= 1) v += __shfl_xor(v, o, 64);
            if (!FWD && g.d_row_w && lane % (CW / 8) == 0 && rbase + j * RPI < row_end) g.d_row_w[rbase + j * RPI] = v;
        }
        if (fr < g.r_pad) {
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int64_t row = row0 + (q & 3) + rgrp + 8 * (q >> 2);
                if (row < row_end) {
                    g.Tg[row * g.ld_t + fr] = to_bf16(acc_g[q] * g.scale);
                    if constexpr (!FWD) g.Tu[row * g.ld_t + fr] = to_bf16(acc_u[q] * g.scale);
                }
            }
        }
        return;
    }
    // the four waves' sums meet in LDS, in wave order (as in small_nt_kernel)
    float* red = (float*)sn_lds;                 // [3 waves][2 products][16][64] floats, over the (now dead) tiles
    __syncthreads();
    if (wave > 0) {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            red[(((wave - 1) * 2 + 0) * 16 + q) * 64 + lane] = acc_g[q];
            red[(((wave - 1) * 2 + 1) * 16 + q) * 64 + lane] = acc_u[q];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int s = 1; s < 4; ++s)
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            acc_g[q] += red[(((s - 1) * 2 + 0) * 16 + q) * 64 + lane];
            acc_u[q] += red[(((s - 1) * 2 + 1) * 16 + q) * 64 + lane];
        }
    if (fr < g.r_pad) {
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int64_t row = row0 + (q & 3) + rgrp + 8 * (q >> 2);
            if (row < row_end) {
                g.Tg[row * g.ld_t + fr] = to_bf16(acc_g[q] * g.scale);
                if constexpr (!FWD) g.Tu[row * g.ld_t + fr] = to_bf16(acc_u[q] * g.scale);
            }
        }
    }
}

template <int FJ, bool GROUPED, bool FWD = false>
static int launch_silu_bwd_nt_one(const SiluNtArgs& g, unsigned blocks, hipStream_t stream) {
    constexpr size_t lds = (size_t)4 * (32 + 32) * (64 + 8) * 2;
    static std::atomic<bool> attr_set{false};   // the attribute call is idempotent: a race only repeats it
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)silu_bwd_nt_kernel<FJ, GROUPED, FWD>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) {
            xq_set_error("silu_bwd_nt: cannot raise the dynamic LDS limit: %s", hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    silu_bwd_nt_kernel<FJ, GROUPED, FWD><<<dim3(blocks), 256, lds, stream>>>(g);
    XQ_CHECK_LAUNCH("silu_bwd_nt");
    return XQ_OK;
}

bool silu_bwd_nt_supported(int64_t cols, int r_pad) { return (r_pad == 16 || r_pad == 32) && cols % 64 == 0 && cols >= 512; }

int launch_silu_bwd_nt(const bf16_t* gate, const bf16_t* up, int64_t ld_gu, const bf16_t* dh, int64_t ld_dh, bf16_t* dgate,
                       bf16_t* dup, int64_t ld_out, int64_t n_rows, int64_t cols, const bf16_t* Fg, const bf16_t* Fu, int r_pad,
                       float scale, bf16_t* Tg, bf16_t* Tu, int64_t ld_t, hipStream_t stream, const int32_t* offsets,
                       const int32_t* tile_offsets, int32_t num_experts, bool shared_fg, bool shared_fu, const float* row_w,
                       float* d_row_w, float swiglu_limit) {
    XQ_REQUIRE(silu_bwd_nt_supported(cols, r_pad), "silu_bwd_nt: %lld columns with r_pad %d are not handled here", (long long)cols, r_pad);
    XQ_REQUIRE(ld_gu % 8 == 0 && ld_dh % 8 == 0 && ld_out % 8 == 0 && ld_t >= r_pad, "silu_bwd_nt: row pitches must be multiples of 8");
    XQ_REQUIRE(xq_aligned(gate, 16) && xq_aligned(up, 16) && xq_aligned(dh, 16) && xq_aligned(dgate, 16) && xq_aligned(dup, 16) &&
                   xq_aligned(Fg, 16) && xq_aligned(Fu, 16),
               "silu_bwd_nt: operands must be 16-byte aligned");
    XQ_REQUIRE(!offsets || (tile_offsets && row_w && num_experts >= 1), "silu_bwd_nt: the routed form needs tile offsets and row weights");
    if (n_rows == 0) return XQ_OK;
    SiluNtArgs g{gate, up, ld_gu, dh, ld_dh, dgate, dup, ld_out, n_rows, cols, Fg, Fu, r_pad, scale, Tg, Tu, ld_t,
                 offsets, tile_offsets, num_experts, offsets && !shared_fg ? (int64_t)r_pad * cols : 0,
                 offsets && !shared_fu ? (int64_t)r_pad * cols : 0, row_w, d_row_w, swiglu_limit};
    if (offsets) {
        const unsigned blocks = (unsigned)(xq_cdiv(n_rows, 128) + num_experts);
        return r_pad == 16 ? launch_silu_bwd_nt_one<4, true>(g, blocks, stream) : launch_silu_bwd_nt_one<8, true>(g, blocks, stream);
    }
    const unsigned blocks = (unsigned)xq_cdiv(n_rows, 32);
    return r_pad == 16 ? launch_silu_bwd_nt_one<4, false>(g, blocks, stream) : launch_silu_bwd_nt_one<8, false>(g, blocks, stream);
}

int launch_silu_fwd_nt(const bf16_t* gate, const bf16_t* up, int64_t ld_gu, bf16_t* h, int64_t ld_h, int64_t n_rows, int64_t cols,
                       const bf16_t* F, int r_pad, float scale, bf16_t* T, int64_t ld_t, hipStream_t stream, const int32_t* offsets,
                       const int32_t* tile_offsets, int32_t num_experts, bool shared_f, const float* row_w, float swiglu_limit) {
    XQ_REQUIRE(silu_bwd_nt_supported(cols, r_pad), "silu_fwd_nt: %lld columns with r_pad %d are not handled here", (long long)cols, r_pad);
    XQ_REQUIRE(ld_gu % 8 == 0 && ld_h % 8 == 0 && ld_t >= r_pad, "silu_fwd_nt: row pitches must be multiples of 8");
    XQ_REQUIRE(xq_aligned(gate, 16) && xq_aligned(up, 16) && xq_aligned(h, 16) && xq_aligned(F, 16), "silu_fwd_nt: operands must be 16-byte aligned");
    XQ_REQUIRE(!offsets || (tile_offsets && row_w && num_experts >= 1), "silu_fwd_nt: the routed form needs tile offsets and row weights");
    if (n_rows == 0) return XQ_OK;
    SiluNtArgs g{gate, up, ld_gu, nullptr, 0, h, nullptr, ld_h, n_rows, cols, F, F, r_pad, scale, T, nullptr, ld_t,
                 offsets, tile_offsets, num_experts, offsets && !shared_f ? (int64_t)r_pad * cols : 0, 0, row_w, nullptr, swiglu_limit};
    if (offsets) {
        const unsigned blocks = (unsigned)(xq_cdiv(n_rows, 128) + num_experts);
        return r_pad == 16 ? launch_silu_bwd_nt_one<4, true, true>(g, blocks, stream) : launch_silu_bwd_nt_one<8, true, true>(g, blocks, stream);
    }
    const unsigned blocks = (unsigned)xq_cdiv(n_rows, 32);
    return r_pad == 16 ? launch_silu_bwd_nt_one<4, false, true>(g, blocks, stream) : launch_silu_bwd_nt_one<8, false, true>(g, blocks, stream);
}

// ------------------------------------------------------------------ tn (weight-gradient shape)
struct TnArgs {
    const bf16_t* P;
    int64_t ldp;
    int64_t width;
    const bf16_t* Q;
    int r_pad, r_out;
    int64_t n_rows;
    int64_t rows_per_split;
    int transpose_out;
    float* out;              // dense: partial [S][width][r_pad]; grouped: out [E][...]
    const int32_t* offsets;  // grouped
    const int32_t* row_limit;  // dense, optional (device): only rows below *row_limit are contracted
    int64_t ldq;               // row pitch of Q in elements
    const int32_t* p_rows;     // optional: row m of the contraction is row p_rows[m] of P
};

constexpr int TN_PP = 128 + 16;  // Ps pitch (bf16 elements): 288 B rows
constexpr int TN_QP = 80;        // Qs pitch: 160 B rows

constexpr int TN_CHUNK = 1024;   // grouped: rows per block (global row chunks, cut at expert boundaries)

// acc += P[m_begin:m_end, c0 + wave*32 .. +32]^T . Q[m_begin:m_end, :]  (m_begin < m_end).  Rows go through LDS 32 at
// a time, in two alternating buffers (Ps, Qs hold both), so one block barrier per tile is enough; the tiles m + 64
// and m + 96 are in flight in registers while tiles m and m + 32 are multiplied.  Every load is unconditional:
// rows past m_end are clamped onto the last row and their Q values replaced by zero, columns past the width are
// clamped onto column 0 and never written.
template <int NT>
__device__ __forceinline__ void tn_accumulate(const TnArgs& g, int64_t c0, int64_t m_begin, int64_t m_end, bf16_t* Ps,
                                              bf16_t* Qs, f32x16* acc) {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pr = tid >> 4, pc = (tid & 15) * 8;  // P tile: rows pr, pr+16; 8 cols at pc
    const int64_t pcol = c0 + pc < g.width ? c0 + pc : 0;   // width % 8 == 0
    const int qchunks = g.r_pad / 8;
    const bool q_thread = tid < 32 * qchunks;
    const int qr = q_thread ? tid / qchunks : 0, qc = q_thread ? (tid % qchunks) * 8 : 0;
    const u32x4 z = {0, 0, 0, 0};
    const int64_t last = m_end - 1;
    struct Tile { u32x4 p0, p1, q; int32_t i0, i1; };
    // with a row map, the P rows of tile m are named by entries fetched one stage earlier (with the data of tile m - 64):
    // the data loads then follow their indices without a round trip of their own in the steady state
    auto fetch_rows = [&](Tile& t, int64_t m) {
        if (g.p_rows) {
            const int64_t r0 = m + pr < m_end ? m + pr : last, r1 = m + pr + 16 < m_end ? m + pr + 16 : last;
            t.i0 = g.p_rows[r0];
            t.i1 = g.p_rows[r1];
        }
    };
    auto fetch = [&](Tile& t, int64_t m) {
        int64_t r0 = m + pr < m_end ? m + pr : last, r1 = m + pr + 16 < m_end ? m + pr + 16 : last;
        const int64_t rq = m + qr < m_end ? m + qr : last;
        if (g.p_rows) { r0 = t.i0; r1 = t.i1; }
        t.p0 = *(const u32x4*)(g.P + r0 * g.ldp + pcol);
        t.p1 = *(const u32x4*)(g.P + r1 * g.ldp + pcol);
        t.q = *(const u32x4*)(g.Q + rq * g.ldq + qc);
        fetch_rows(t, m + 64);
    };
    auto tile = [&](Tile& t, int64_t m, int buf) {     // multiply tile m out of LDS buffer `buf`, refill t with tile m + 64
        bf16_t* ps = Ps + buf * (32 * TN_PP);
        bf16_t* qs = Qs + buf * (32 * TN_QP);
        *(u32x4*)(ps + pr * TN_PP + pc) = t.p0;
        *(u32x4*)(ps + (pr + 16) * TN_PP + pc) = t.p1;
        if (q_thread) *(u32x4*)(qs + qr * TN_QP + qc) = m + qr < m_end ? t.q : z;
        fetch(t, m + 64);
        // the other buffer's fragment reads lie before this barrier in every wave, its next stores after the next one
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8 a = lds_tr_frag(ps, TN_PP, ks * 16, wave * 32, lane);
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                bf16x8 b = lds_tr_frag(qs, TN_QP, ks * 16, n * 32, lane);
                acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[n], 0, 0, 0);
            }
        }
    };
    Tile ta, tb;
    fetch_rows(ta, m_begin);
    fetch_rows(tb, m_begin + 32);
    fetch(ta, m_begin);
    fetch(tb, m_begin + 32);
    for (int64_t m = m_begin; m < m_end; m += 64) {
        tile(ta, m, 0);
        tile(tb, m + 32, 1);        // past m_end: all-zero Q rows, no contribution
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // the buffers are free again when this returns
}

// out[c][j] (pitch = row length of the destination) or, transposed, out[j][c]; j < r_lim
template <int NT>
__device__ __forceinline__ void tn_write(const f32x16* acc, float* out, int64_t c0, int64_t width, int r_lim, int pitch,
                                         bool transposed) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int rgrp = (lane >> 5) * 4;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        const int j = n * 32 + (lane & 31);
        if (j >= r_lim) continue;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const int64_t c = c0 + wave * 32 + (q & 3) + rgrp + 8 * (q >> 2);
            if (c >= width) continue;
            if (transposed) out[(int64_t)j * width + c] = acc[n][q];
            else out[c * pitch + j] = acc[n][q];
        }
    }
}

// dense: block (col tile, row split) -> partial[split][width][r_pad]
template <int NT>
__global__ void __launch_bounds__(256) tn_kernel(TnArgs g) {
    __shared__ __attribute__((aligned(16))) bf16_t Ps[2 * 32 * TN_PP];
    __shared__ __attribute__((aligned(16))) bf16_t Qs[2 * 32 * TN_QP];
    const int64_t c0 = (int64_t)blockIdx.x * 128;
    const int64_t m_begin = (int64_t)blockIdx.y * g.rows_per_split;
    int64_t m_end = m_begin + g.rows_per_split;
    m_end = m_end < g.n_rows ? m_end : g.n_rows;
    if (g.row_limit) {
        const int64_t lim = *g.row_limit;
        m_end = m_end < lim ? m_end : lim;
    }
    f32x16 acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[n][q] = 0.0f;
    if (m_begin < m_end) tn_accumulate<NT>(g, c0, m_begin, m_end, Ps, Qs, acc);     // uniform over the block
    tn_write<NT>(acc, g.out + (int64_t)blockIdx.y * g.width * g.r_pad, c0, g.width, g.r_pad, g.r_pad, false);
}

// grouped: block (col tile, chunk of TN_CHUNK global rows).  The chunk is walked expert by expert;
// an expert that lies wholly inside the chunk is written to out[e] directly, a piece of an expert
// that continues from the previous chunk goes to partial[chunk][0], one that continues into the
// next chunk to partial[chunk][1] (tn_grouped_reduce_kernel adds the pieces in chunk order).
template <int NT>
__global__ void __launch_bounds__(256) tn_grouped_kernel(TnArgs g, int32_t num_experts, float* partial) {
    __shared__ __attribute__((aligned(16))) bf16_t Ps[2 * 32 * TN_PP];
    __shared__ __attribute__((aligned(16))) bf16_t Qs[2 * 32 * TN_QP];
    __shared__ int sh_e;
    const int64_t c0 = (int64_t)blockIdx.x * 128;
    const int64_t r_begin = (int64_t)blockIdx.y * TN_CHUNK;
    int64_t r_end = r_begin + TN_CHUNK;
    r_end = r_end < g.n_rows ? r_end : g.n_rows;
    // the expert that owns row r_begin (offsets[e] <= r_begin < offsets[e + 1]; r_begin < n_rows = offsets[E], so
    // exactly one does): one look per thread instead of a chain of dependent loads
    if (threadIdx.x == 0) sh_e = num_experts;      // rows beyond the last expert's: nothing to do
    __syncthreads();
    for (int x = threadIdx.x; x < num_experts; x += 256) {
        const int64_t o0 = g.offsets[x], o1 = g.offsets[x + 1];
        if (o0 <= r_begin && r_begin < o1) sh_e = x;
    }
    __syncthreads();
    int e = sh_e;
    int64_t m = r_begin;
    while (m < r_end && e < num_experts) {
        const int64_t eb = g.offsets[e], ee = g.offsets[e + 1];
        const int64_t seg_end = ee < r_end ? ee : r_end;
        if (seg_end <= m) { ++e; continue; }   // expert without rows (or already passed)
        f32x16 acc[NT];
#pragma unroll
        for (int n = 0; n < NT; ++n)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[n][q] = 0.0f;
        tn_accumulate<NT>(g, c0, m, seg_end, Ps, Qs, acc);
        if (eb >= r_begin && ee <= r_end)
            tn_write<NT>(acc, g.out + (int64_t)e * g.width * g.r_out, c0, g.width, g.r_out, g.r_out, g.transpose_out != 0);
        else
            tn_write<NT>(acc, partial + ((int64_t)blockIdx.y * 2 + (eb < r_begin ? 0 : 1)) * g.width * g.r_pad, c0, g.width,
                         g.r_pad, g.r_pad, false);
        m = seg_end;
        ++e;
    }
}

// out[e] for the experts the chunk walk did not finish: zero for an expert without rows, the sum of
// its pieces in chunk order for one that spans several chunks.
__global__ void __launch_bounds__(256) tn_grouped_reduce_kernel(const float* partial, const int32_t* offsets, int64_t width,
                                                                int r_pad, int r_out, int transpose_out, float* out) {
    const int e = blockIdx.y;
    const int64_t b = offsets[e], en = offsets[e + 1];
    const int64_t ch0 = b / TN_CHUNK, ch1 = en > b ? (en - 1) / TN_CHUNK : ch0;
    if (en > b && ch0 == ch1) return;   // written directly
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= width * r_pad) return;
    const int64_t c = t / r_pad;
    const int j = (int)(t - c * r_pad);
    if (j >= r_out) return;
    float s = 0.0f;
    if (en > b) {
        const int64_t per = width * r_pad;
        s = partial[(ch0 * 2 + 1) * per + t];
        for (int64_t ch = ch0 + 1; ch <= ch1; ++ch) s += partial[(ch * 2) * per + t];
    }
    float* o = out + (int64_t)e * width * r_out;
    if (transpose_out) o[(int64_t)j * width + c] = s;
    else o[c * r_out + j] = s;
}

// sums the dense partials in split order: out[c][j] or out[j][c], j < r_out
__global__ void __launch_bounds__(256) tn_reduce_kernel(const float* partial, int splits, int64_t width, int r_pad,
                                                        int r_out, int transpose_out, float* out) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= width * r_pad) return;
    int64_t c = t / r_pad;
    int j = (int)(t - c * r_pad);
    if (j >= r_out) return;
    float s = 0.0f;
    for (int i = 0; i < splits; ++i) s += partial[(int64_t)i * width * r_pad + t];
    if (transpose_out) out[(int64_t)j * width + c] = s;
    else out[c * r_out + j] = s;
}

static int tn_splits(int64_t n_rows, int64_t width) {
    int64_t col_tiles = xq_cdiv(width, 128);
    int64_t s = xq_cdiv(768, col_tiles);
    int64_t max_s = n_rows / 256 > 0 ? n_rows / 256 : 1;
    if (s > max_s) s = max_s;
    if (s > 32) s = 32;
    return (int)(s < 1 ? 1 : s);
}

int64_t tn_partial_bytes(int64_t n_rows, int64_t width, int r_pad) {
    const int64_t dense = (int64_t)tn_splits(n_rows, width) * width * r_pad * 4;
    const int64_t grouped = xq_cdiv(n_rows > 0 ? n_rows : 1, TN_CHUNK) * 2 * width * r_pad * 4;
    return dense > grouped ? dense : grouped;
}

int launch_tn(const bf16_t* P, int64_t ldp, int64_t width, const bf16_t* Q, int r_pad, int r_out, int64_t n_rows,
              bool transpose_out, float* out, float* partial, const int32_t* offsets, int32_t num_experts,
              hipStream_t stream, const int32_t* row_limit, int64_t ldq, const int32_t* p_rows) {
    if (ldq <= 0) ldq = r_pad;
    XQ_REQUIRE(ldq >= r_pad && ldq % 8 == 0, "tn: Q pitch %lld must be a multiple of 8 and at least r_pad", (long long)ldq);
    XQ_REQUIRE(r_pad > 0 && r_pad <= 64 && r_pad % 16 == 0 && r_out <= r_pad, "tn: bad rank (r_pad %d, r_out %d)", r_pad, r_out);
    XQ_REQUIRE(width % 8 == 0 && ldp % 8 == 0 && xq_aligned(P, 16) && xq_aligned(Q, 16), "tn: operands must be 16-byte aligned, width %% 8 == 0");
    if (width == 0 || r_out == 0) return XQ_OK;
    TnArgs g{P, ldp, width, Q, r_pad, r_out, n_rows, 0, transpose_out ? 1 : 0, out, offsets, offsets ? nullptr : row_limit, ldq, p_rows};
    unsigned col_tiles = (unsigned)xq_cdiv(width, 128);
    XQ_REQUIRE(partial != nullptr, "tn: partial workspace is NULL");
    if (offsets) {
        if (n_rows > 0) {
            dim3 grid(col_tiles, (unsigned)xq_cdiv(n_rows, TN_CHUNK));
            if (r_pad <= 32) tn_grouped_kernel<1><<<grid, 256, 0, stream>>>(g, num_experts, partial);
            else tn_grouped_kernel<2><<<grid, 256, 0, stream>>>(g, num_experts, partial);
            XQ_CHECK_LAUNCH("tn(grouped)");
        }
        dim3 rgrid((unsigned)xq_cdiv(width * r_pad, 256), (unsigned)num_experts);
        tn_grouped_reduce_kernel<<<rgrid, 256, 0, stream>>>(partial, offsets, width, r_pad, r_out, transpose_out ? 1 : 0, out);
        XQ_CHECK_LAUNCH("tn(grouped reduce)");
        return XQ_OK;
    }
    int S = tn_splits(n_rows, width);
    int64_t rps = xq_cdiv(xq_cdiv(n_rows, S), 32) * 32;
    g.rows_per_split = rps;
    g.out = partial;
    dim3 grid(col_tiles, (unsigned)S);
    if (r_pad <= 32) tn_kernel<1><<<grid, 256, 0, stream>>>(g);
    else tn_kernel<2><<<grid, 256, 0, stream>>>(g);
    XQ_CHECK_LAUNCH("tn");
    tn_reduce_kernel<<<dim3((unsigned)xq_cdiv(width * r_pad, 256)), 256, 0, stream>>>(partial, S, width, r_pad, r_out,
                                                                                      transpose_out ? 1 : 0, out);
    XQ_CHECK_LAUNCH("tn_reduce");
    return XQ_OK;
}

}  // namespace xq
