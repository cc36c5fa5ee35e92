// Low-rank helper kernels (see xq_lora.h).  bf16 MFMA, fp32 accumulate.
#include "xq_lora.h"

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
    const int32_t* offsets;
    const int32_t* tile_offsets;
    int32_t num_experts;
};

// TR rows per block: 32 (dense; the 4 waves split K) or 128 (grouped; one wave per 32 rows).
template <int TR, int NT>
__global__ void __launch_bounds__(256) small_nt_kernel(SmallNtArgs g) {
    constexpr int RG = TR / 32, KS = 4 / RG;
    __shared__ float red[KS > 1 ? (KS - 1) * NT * 64 * 16 : 1];
    __shared__ int sh_info[3];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int rg = wave % RG, ks = wave / RG;

    int e = 0;
    int64_t row0, row_end;
    if (g.offsets) {
        if (tid == 0) {
            int t = blockIdx.x, lo = 0, hi = g.num_experts;
            if (t >= g.tile_offsets[g.num_experts]) sh_info[0] = -1;
            else {
                while (hi - lo > 1) { int mid = (lo + hi) >> 1; if (g.tile_offsets[mid] <= t) lo = mid; else hi = mid; }
                sh_info[0] = lo;
                sh_info[1] = g.offsets[lo] + (t - g.tile_offsets[lo]) * TR;
                sh_info[2] = g.offsets[lo + 1];
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
    const int fr = lane & 31, fk = (lane >> 5) * 8;
    int64_t arow = row0 + rg * 32 + fr;
    arow = arow < row_end ? arow : row_end - 1;
    const bf16_t* ap = g.In + arow * g.ld_in + fk;
    const bf16_t* fp[NT];
    bool fvalid[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        int j = n * 32 + fr;
        fvalid[n] = j < g.r_pad;
        fp[n] = F + (int64_t)(fvalid[n] ? j : 0) * g.Kc + fk;
    }
    f32x16 acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[n][q] = 0.0f;

    const int64_t kspan = g.Kc / KS;  // multiple of 16
    const int64_t kbeg = ks * kspan, kend = kbeg + kspan;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    int64_t k = kbeg;
    for (; k + 64 <= kend; k += 64) {
        bf16x8 a[4], b[NT][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            a[u] = *(const bf16x8*)(ap + k + u * 16);
#pragma unroll
            for (int n = 0; n < NT; ++n) b[n][u] = fvalid[n] ? *(const bf16x8*)(fp[n] + k + u * 16) : zero8;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
#pragma unroll
            for (int n = 0; n < NT; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[u], b[n][u], acc[n], 0, 0, 0);
    }
    for (; k < kend; k += 16) {
        bf16x8 a = *(const bf16x8*)(ap + k);
#pragma unroll
        for (int n = 0; n < NT; ++n) {
            bf16x8 b = fvalid[n] ? *(const bf16x8*)(fp[n] + k) : zero8;
            acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[n], 0, 0, 0);
        }
    }

    if (KS > 1) {
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
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            int64_t row = row0 + rg * 32 + (q & 3) + rgrp + 8 * (q >> 2);
            if (row < row_end) g.T[row * g.r_pad + j] = to_bf16(acc[n][q] * g.scale);
        }
    }
}

int launch_small_nt(const bf16_t* In, int64_t ld_in, int64_t n_rows, int64_t Kc, const bf16_t* F, int r_pad,
                    float scale, bf16_t* T, const int32_t* offsets, const int32_t* tile_offsets,
                    int32_t num_experts, bool shared_f, hipStream_t stream) {
    XQ_REQUIRE(r_pad > 0 && r_pad <= 64 && r_pad % 16 == 0, "small_nt: r_pad must be 16/32/48/64, got %d", r_pad);
    XQ_REQUIRE(Kc % 64 == 0, "small_nt: contraction length %lld must be a multiple of 64", (long long)Kc);
    XQ_REQUIRE(ld_in % 8 == 0 && xq_aligned(In, 16) && xq_aligned(F, 16), "small_nt: operands must be 16-byte aligned");
    if (n_rows == 0) return XQ_OK;
    SmallNtArgs g{In, ld_in, n_rows, Kc, F, shared_f ? 0 : (int64_t)r_pad * Kc, r_pad, scale, T, offsets, tile_offsets,
                  num_experts};
    if (offsets) {
        unsigned blocks = (unsigned)(xq_cdiv(n_rows, 128) + num_experts);
        if (r_pad <= 32) small_nt_kernel<128, 1><<<dim3(blocks), 256, 0, stream>>>(g);
        else small_nt_kernel<128, 2><<<dim3(blocks), 256, 0, stream>>>(g);
    } else {
        g.f_stride = 0;
        unsigned blocks = (unsigned)xq_cdiv(n_rows, 32);
        if (r_pad <= 32) small_nt_kernel<32, 1><<<dim3(blocks), 256, 0, stream>>>(g);
        else small_nt_kernel<32, 2><<<dim3(blocks), 256, 0, stream>>>(g);
    }
    XQ_CHECK_LAUNCH("small_nt");
    return XQ_OK;
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
};

constexpr int TN_PP = 128 + 16;  // Ps pitch (bf16 elements): 288 B rows
constexpr int TN_QP = 80;        // Qs pitch: 160 B rows

template <int NT>
__global__ void __launch_bounds__(256) tn_kernel(TnArgs g) {
    __shared__ __attribute__((aligned(16))) bf16_t Ps[32 * TN_PP];
    __shared__ __attribute__((aligned(16))) bf16_t Qs[32 * TN_QP];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t c0 = (int64_t)blockIdx.x * 128;
    int64_t m_begin, m_end;
    float* out;
    if (g.offsets) {
        m_begin = g.offsets[blockIdx.y];
        m_end = g.offsets[blockIdx.y + 1];
        out = g.out + (int64_t)blockIdx.y * g.width * g.r_out;
    } else {
        m_begin = (int64_t)blockIdx.y * g.rows_per_split;
        m_end = m_begin + g.rows_per_split;
        m_end = m_end < g.n_rows ? m_end : g.n_rows;
        out = g.out + (int64_t)blockIdx.y * g.width * g.r_pad;
    }
    f32x16 acc[NT];
#pragma unroll
    for (int n = 0; n < NT; ++n)
#pragma unroll
        for (int q = 0; q < 16; ++q) acc[n][q] = 0.0f;

    const int pr = tid >> 4, pc = (tid & 15) * 8;  // P tile: rows pr, pr+16; 8 cols at pc
    const bool pcol_ok = c0 + pc < g.width;        // width % 8 == 0
    const int qchunks = g.r_pad / 8;
    const int qr = tid / qchunks, qc = (tid % qchunks) * 8;
    const bool q_thread = tid < 32 * qchunks;
    const u32x4 z = {0, 0, 0, 0};

    for (int64_t m = m_begin; m < m_end; m += 32) {
        u32x4 p0 = z, p1 = z, qv = z;
        if (pcol_ok) {
            if (m + pr < m_end) p0 = *(const u32x4*)(g.P + (m + pr) * g.ldp + c0 + pc);
            if (m + pr + 16 < m_end) p1 = *(const u32x4*)(g.P + (m + pr + 16) * g.ldp + c0 + pc);
        }
        if (q_thread && m + qr < m_end) qv = *(const u32x4*)(g.Q + (m + qr) * g.r_pad + qc);
        __syncthreads();  // previous iteration's fragment reads are done
        *(u32x4*)(Ps + pr * TN_PP + pc) = p0;
        *(u32x4*)(Ps + (pr + 16) * TN_PP + pc) = p1;
        if (q_thread) *(u32x4*)(Qs + qr * TN_QP + qc) = qv;
        __syncthreads();
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            bf16x8 a = lds_tr_frag(Ps, TN_PP, ks * 16, wave * 32, lane);
#pragma unroll
            for (int n = 0; n < NT; ++n) {
                bf16x8 b = lds_tr_frag(Qs, TN_QP, ks * 16, n * 32, lane);
                acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[n], 0, 0, 0);
            }
        }
    }
    const int rgrp = (lane >> 5) * 4;
#pragma unroll
    for (int n = 0; n < NT; ++n) {
        int j = n * 32 + (lane & 31);
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            int64_t c = c0 + wave * 32 + (q & 3) + rgrp + 8 * (q >> 2);
            if (c >= g.width) continue;
            if (g.offsets) {
                if (j < g.r_out) {
                    if (g.transpose_out) out[(int64_t)j * g.width + c] = acc[n][q];
                    else out[c * g.r_out + j] = acc[n][q];
                }
            } else if (j < g.r_pad) {
                out[c * g.r_pad + j] = acc[n][q];
            }
        }
    }
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
    return (int64_t)tn_splits(n_rows, width) * width * r_pad * 4;
}

int launch_tn(const bf16_t* P, int64_t ldp, int64_t width, const bf16_t* Q, int r_pad, int r_out, int64_t n_rows,
              bool transpose_out, float* out, float* partial, const int32_t* offsets, int32_t num_experts,
              hipStream_t stream) {
    XQ_REQUIRE(r_pad > 0 && r_pad <= 64 && r_pad % 16 == 0 && r_out <= r_pad, "tn: bad rank (r_pad %d, r_out %d)", r_pad, r_out);
    XQ_REQUIRE(width % 8 == 0 && ldp % 8 == 0 && xq_aligned(P, 16) && xq_aligned(Q, 16), "tn: operands must be 16-byte aligned, width %% 8 == 0");
    if (width == 0 || r_out == 0) return XQ_OK;
    TnArgs g{P, ldp, width, Q, r_pad, r_out, n_rows, 0, transpose_out ? 1 : 0, out, offsets};
    unsigned col_tiles = (unsigned)xq_cdiv(width, 128);
    if (offsets) {
        dim3 grid(col_tiles, (unsigned)num_experts);
        if (r_pad <= 32) tn_kernel<1><<<grid, 256, 0, stream>>>(g);
        else tn_kernel<2><<<grid, 256, 0, stream>>>(g);
        XQ_CHECK_LAUNCH("tn(grouped)");
        return XQ_OK;
    }
    XQ_REQUIRE(partial != nullptr, "tn: partial workspace is NULL");
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
