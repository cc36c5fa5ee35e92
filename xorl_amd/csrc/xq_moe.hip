// SwiGLU (dense and routed) and the token <-> expert-order permutation kernels.
//   SwiGLU      ops/fused_silu_and_mul.py:22-60 (two roundings); routed form
//               ops/moe/lora.py:639-647 (silu -> *up -> *routing weight, bf16 each)
//   routing     ops/moe/lora.py:579-583 (histogram, stable argsort, cumsum)
//   scatter     ops/group_gemm/kernel/moe.py:266-312
//   gather      ops/group_gemm/kernel/moe.py:102-141 (fp32 accumulate), :178-223 (add_gather)
#include "xq_common.h"
#include <atomic>

namespace {

// h = bf16(bf16(bf16(silu(g)) * u) * w_row)
__global__ void __launch_bounds__(256) silu_mul_fwd_kernel(const bf16_t* gate, const bf16_t* up, int64_t ld_in,
                                                           const float* row_w, bf16_t* h, int64_t ld_h, int64_t rows,
                                                           int64_t cols8, float limit) {
    int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= rows * cols8) return;
    int64_t r = t / cols8, c = (t - r * cols8) * 8;
    u32x4 gv = *(const u32x4*)(gate + r * ld_in + c), uv = *(const u32x4*)(up + r * ld_in + c);
    float w = row_w ? row_w[r] : 1.0f;
    u32x4 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float res[2];
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf) {
            float g = bf16_to_f32((bf16_t)(gv[i] >> (16 * hlf))), u = bf16_to_f32((bf16_t)(uv[i] >> (16 * hlf)));
            g = swiglu_clamp(g, limit);
            float a = round_bf16(g * sigmoid_f32(g));
            float v = a * u;
            if (row_w) v = round_bf16(v) * w;
            res[hlf] = v;
        }
        o[i] = pack_bf16x2(res[0], res[1]);
    }
    *(u32x4*)(h + r * ld_h + c) = o;
}

// Given dh = d(loss)/d(h):  with a = bf16(silu(g)), p = a*u, h = p*w
//   dp = dh*w ; dgate = dp*u*silu'(g) ; dup = dp*a ; dw[row] = sum_c dh*p
// (ops/moe/lora.py:855-917; silu'(g) = s*(1+g*(1-s)), aten.silu_backward)
__global__ void __launch_bounds__(256) silu_mul_bwd_kernel(const bf16_t* gate, const bf16_t* up, int64_t ld_in,
                                                           const bf16_t* dh, int64_t ld_dh, const float* row_w,
                                                           bf16_t* dgate, bf16_t* dup, int64_t ld_out, float* d_row_w,
                                                           int64_t rows, int64_t cols, float limit) {
    // one block per row (cols/8 vector steps striding over the row) so the row-weight gradient is a block reduction
    __shared__ float red[4];
    const int64_t r = blockIdx.x;
    const float w = row_w ? row_w[r] : 1.0f;
    float wsum = 0.0f;
    for (int64_t c = (int64_t)threadIdx.x * 8; c < cols; c += 256 * 8) {
        u32x4 gv = *(const u32x4*)(gate + r * ld_in + c), uv = *(const u32x4*)(up + r * ld_in + c);
        u32x4 dv = *(const u32x4*)(dh + r * ld_dh + c);
        u32x4 og, ou;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float rg[2], ru[2];
#pragma unroll
            for (int hlf = 0; hlf < 2; ++hlf) {
                float g = bf16_to_f32((bf16_t)(gv[i] >> (16 * hlf))), u = bf16_to_f32((bf16_t)(uv[i] >> (16 * hlf)));
                float d = bf16_to_f32((bf16_t)(dv[i] >> (16 * hlf)));
                const float open = swiglu_mask(g, limit);
                g = swiglu_clamp(g, limit);
                float s = sigmoid_f32(g);
                float a = round_bf16(g * s);
                float dp = row_w ? round_bf16(d * w) : d;
                wsum += d * round_bf16(a * u);
                rg[hlf] = round_bf16(dp * u) * (s * (1.0f + g * (1.0f - s))) * open;
                ru[hlf] = a * dp;
            }
            og[i] = pack_bf16x2(rg[0], rg[1]);
            ou[i] = pack_bf16x2(ru[0], ru[1]);
        }
        *(u32x4*)(dgate + r * ld_out + c) = og;
        *(u32x4*)(dup + r * ld_out + c) = ou;
    }
    if (d_row_w) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) wsum += __shfl_down(wsum, o, 64);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = wsum;
        __syncthreads();
        if (threadIdx.x == 0) d_row_w[r] = (red[0] + red[1]) + (red[2] + red[3]);
    }
}

// ------------------------------------------------------------------ routing
constexpr int RB_CHUNK = 256;   // routed entries per block (one wave walks them in order)
constexpr int RB_MAX_E = 1024;

// pass 1: per-chunk histogram
__global__ void __launch_bounds__(64) route_hist_kernel(const int32_t* sel, int64_t n, int32_t E, int32_t* chunk_counts) {
    __shared__ int32_t cnt[RB_MAX_E];
    for (int e = threadIdx.x; e < E; e += 64) cnt[e] = 0;
    __syncthreads();
    int64_t base = (int64_t)blockIdx.x * RB_CHUNK;
    for (int i = threadIdx.x; i < RB_CHUNK; i += 64) {
        int64_t idx = base + i;
        if (idx < n) {
            int e = sel[idx];
            if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < E; e += 64) chunk_counts[(int64_t)blockIdx.x * E + e] = cnt[e];
}

// pass 2 (one block of 16 waves): totals, expert offsets, tile offsets, and per-chunk bases (exclusive scan over
// chunks).  The counts are a [chunk][expert] matrix; wave w owns the chunk rows [w * cpw, (w + 1) * cpw) and its
// lanes the experts (a row is read with coalesced loads, eight rows in flight): column sums of the wave's rows,
// then, through LDS, each wave's base = the sums of the waves before it, then the running base written back over
// the counts.  The prefixes over experts are one wave's scans, 64 experts at a time.
__device__ __forceinline__ int32_t wave_inclusive_scan(int32_t v, int lane) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const int32_t u = __shfl_up(v, o, 64);
        if (lane >= o) v += u;
    }
    return v;
}

__global__ void __launch_bounds__(1024) route_scan_kernel(int32_t* chunk_counts, int32_t n_chunks, int32_t E,
                                                          int32_t* counts, int32_t* offsets, int32_t* tile_offsets) {
    extern __shared__ int32_t scan_lds[];
    int32_t* part = scan_lds;            // [16][E]
    int32_t* tot = scan_lds + 16 * E;    // [E]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cpw = (n_chunks + 15) >> 4;
    const int c_begin = wave * cpw, c_end = c_begin + cpw < n_chunks ? c_begin + cpw : n_chunks;
    const int c_last = n_chunks - 1;
    for (int e = lane; e < E; e += 64) {
        int32_t sum = 0;
        for (int c = c_begin; c < c_end; c += 8) {
            int32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = chunk_counts[(int64_t)(c + u < c_end ? c + u : c_last) * E + e];
#pragma unroll
            for (int u = 0; u < 8; ++u) sum += c + u < c_end ? v[u] : 0;
        }
        part[wave * E + e] = sum;
    }
    __syncthreads();
    for (int e = lane; e < E; e += 64) {
        int32_t run = 0, total = 0;
        for (int w = 0; w < 16; ++w) {
            const int32_t v = part[w * E + e];
            run += w < wave ? v : 0;
            total += v;
        }
        if (wave == 0) {
            tot[e] = total;
            counts[e] = total;
        }
        for (int c = c_begin; c < c_end; c += 8) {
            int32_t v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = chunk_counts[(int64_t)(c + u < c_end ? c + u : c_last) * E + e];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (c + u < c_end) {
                    chunk_counts[(int64_t)(c + u) * E + e] = run;   // becomes the chunk's base within the expert
                    run += v[u];
                }
            }
        }
    }
    __syncthreads();
    if (wave == 0) {
        int32_t o = 0, t = 0, t2 = 0;
        int32_t* tiles256 = tile_offsets + (E + 1);
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int32_t c = e < E ? tot[e] : 0;
            const int32_t c128 = (c + 127) / 128, c256 = (c + 255) / 256;
            const int32_t io = wave_inclusive_scan(c, lane), it = wave_inclusive_scan(c128, lane), it2 = wave_inclusive_scan(c256, lane);
            if (e < E) {
                offsets[e] = o + io - c;
                tile_offsets[e] = t + it - c128;
                tiles256[e] = t2 + it2 - c256;
            }
            o += __shfl(io, 63, 64);
            t += __shfl(it, 63, 64);
            t2 += __shfl(it2, 63, 64);
        }
        if (lane == 0) {
            offsets[E] = o;
            tile_offsets[E] = t;
            tiles256[E] = t2;
        }
    }
}

// pass 3: stable position of every routed entry (one wave per chunk, in order).  The lanes of a 64-entry segment that
// hold the same expert are found by intersecting, over the bits of the expert id, the ballots of "my value of
// this bit"; a lane's position is the expert's running base plus the number of such lanes below it.
__global__ void __launch_bounds__(64) route_place_kernel(const int32_t* sel, int64_t n, int32_t E, int32_t id_bits,
                                                         const int32_t* chunk_base, const int32_t* offsets,
                                                         int32_t* scatter_index) {
    __shared__ int32_t run[RB_MAX_E];
    for (int e = threadIdx.x; e < E; e += 64) run[e] = offsets[e] + chunk_base[(int64_t)blockIdx.x * E + e];
    __syncthreads();
    const int lane = threadIdx.x;
    const uint64_t below = (1ull << lane) - 1ull;
    int64_t base = (int64_t)blockIdx.x * RB_CHUNK;
    for (int seg = 0; seg < RB_CHUNK; seg += 64) {
        int64_t idx = base + seg + lane;
        bool valid = idx < n;
        int e = valid ? sel[idx] : -1;
        if (e >= E) e = -1;
        uint64_t same = __ballot(e >= 0);
        for (int b = 0; b < id_bits; ++b) {
            const bool bit = (e >> b) & 1;
            const uint64_t m = __ballot(bit);
            same &= bit ? m : ~m;
        }
        const int before = __popcll(same & below);
        const bool last = (same & ~below & ~(1ull << lane)) == 0;   // no higher lane holds this expert
        if (e >= 0) scatter_index[idx] = run[e] + before;
        else if (valid) scatter_index[idx] = -1;          // id outside [0, E): the copy is dropped by every consumer
        __syncthreads();
        if (e >= 0 && last) run[e] += before + 1;
        __syncthreads();
    }
}

// out[scatter_index[t * topk + j]] = in[t] for j < topk (rows of `width` bf16; width % 8 == 0).  One block per
// token: the source row is read once and stored topk times, so the kernel runs at the rate of its writes.
__global__ void __launch_bounds__(256) moe_scatter_kernel(const bf16_t* in, int64_t ld_in, const int32_t* sidx,
                                                          int32_t topk, int64_t width8, bf16_t* out, int64_t ld_out) {
    const int64_t t = blockIdx.x;
    const u32x4* src = (const u32x4*)(in + t * ld_in);
    const int32_t* dst_rows = sidx + t * topk;             // uniform: scalar loads
    for (int64_t c = threadIdx.x; c < width8; c += 256) {
        const u32x4 v = src[c];
        for (int j0 = 0; j0 < topk; j0 += 8) {
            int64_t r[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) r[u] = dst_rows[j0 + u < topk ? j0 + u : topk - 1];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (j0 + u < topk && r[u] >= 0) ((u32x4*)(out + r[u] * ld_out))[c] = v;     // uniform; -1 = dropped copy
        }
    }
}

// dst[scatter_index[i]] = src[i] (fp32 scalars; routing weights bf16/fp32 -> fp32)
__global__ void __launch_bounds__(256) moe_scatter_scalar_kernel(const void* src, int src_f32, const int32_t* sidx,
                                                                 int64_t n, float* dst) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int32_t d = sidx[i];
    if (d < 0) return;                                   // dropped copy
    dst[d] = src_f32 ? ((const float*)src)[i] : bf16_to_f32(((const bf16_t*)src)[i]);
}
// dst[i] = src[scatter_index[i]]
__global__ void __launch_bounds__(256) moe_gather_scalar_kernel(const float* src, const int32_t* sidx, int64_t n,
                                                                void* dst, int dst_f32) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int32_t d = sidx[i];
    float v = d < 0 ? 0.0f : src[d];                     // a dropped copy has no row: zero
    if (dst_f32) ((float*)dst)[i] = v;
    else ((bf16_t*)dst)[i] = to_bf16(v);
}

// out[t] = sum_j rows[sidx[t*topk+j]] (+ rows2[...]); fp32 accumulate in slot order.  One block per token; the row
// indices of up to 8 slots are fetched first and their loads issued together (slots past topk are clamped onto
// the last one and their values left out), so a token costs one memory round trip instead of one per slot.
template <bool TWO>
__global__ void __launch_bounds__(256) moe_gather_kernel(const bf16_t* rows, const bf16_t* rows2, int64_t ld_rows,
                                                         const int32_t* sidx, int32_t topk, int64_t width8,
                                                         bf16_t* out, int64_t ld_out) {
    const int64_t t = blockIdx.x;
    const int32_t* src_rows = sidx + t * topk;             // uniform: scalar loads
    for (int64_t c = threadIdx.x; c < width8; c += 256) {
        float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int j0 = 0; j0 < topk; j0 += 8) {
            u32x4 v[8], v2[8];
            bool keep[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int64_t r0 = src_rows[j0 + u < topk ? j0 + u : topk - 1];
                keep[u] = r0 >= 0;                         // -1 = dropped copy: row 0 is read in its place and left out
                const int64_t r = keep[u] ? r0 : 0;
                v[u] = ((const u32x4*)(rows + r * ld_rows))[c];
                if (TWO) v2[u] = ((const u32x4*)(rows2 + r * ld_rows))[c];
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                if (j0 + u < topk && keep[u]) {            // uniform
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        acc[2 * q] += bf16_to_f32((bf16_t)(v[u][q] & 0xffffu));
                        acc[2 * q + 1] += bf16_to_f32((bf16_t)(v[u][q] >> 16));
                    }
                    if (TWO) {
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            acc[2 * q] += bf16_to_f32((bf16_t)(v2[u][q] & 0xffffu));
                            acc[2 * q + 1] += bf16_to_f32((bf16_t)(v2[u][q] >> 16));
                        }
                    }
                }
            }
        }
        ((u32x4*)(out + t * ld_out))[c] = u32x4{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3]),
                                                pack_bf16x2(acc[4], acc[5]), pack_bf16x2(acc[6], acc[7])};
    }
}

}  // namespace

namespace xq {
int silu_mul_fwd_limit(const void* gate, const void* up, int64_t ld_in, const float* row_w, void* h, int64_t ld_h, int64_t rows,
                       int64_t cols, float limit, void* stream) {
    XQ_REQUIRE(cols % 8 == 0 && ld_in % 8 == 0 && ld_h % 8 == 0, "xq_silu_mul_fwd: cols and strides must be multiples of 8");
    if (rows == 0 || cols == 0) return XQ_OK;   // an empty batch has no storage to point at
    XQ_REQUIRE(gate && up && h, "xq_silu_mul_fwd: NULL pointer");
    XQ_REQUIRE(xq_aligned(gate, 16) && xq_aligned(up, 16) && xq_aligned(h, 16), "xq_silu_mul_fwd: pointers must be 16-byte aligned");
    int64_t total = rows * (cols / 8);
    silu_mul_fwd_kernel<<<dim3((unsigned)xq_cdiv(total, 256)), 256, 0, (hipStream_t)stream>>>(
        (const bf16_t*)gate, (const bf16_t*)up, ld_in, row_w, (bf16_t*)h, ld_h, rows, cols / 8, limit);
    XQ_CHECK_LAUNCH("xq_silu_mul_fwd");
    return XQ_OK;
}

int silu_mul_bwd_limit(const void* gate, const void* up, int64_t ld_in, const void* dh, int64_t ld_dh, const float* row_w, void* dgate,
                       void* dup, int64_t ld_out, float* d_row_w, int64_t rows, int64_t cols, float limit, void* stream) {
    XQ_REQUIRE(cols % 8 == 0 && ld_in % 8 == 0 && ld_dh % 8 == 0 && ld_out % 8 == 0, "xq_silu_mul_bwd: cols and strides must be multiples of 8");
    if (rows == 0 || cols == 0) return XQ_OK;   // an empty batch has no storage to point at
    XQ_REQUIRE(gate && up && dh && dgate && dup, "xq_silu_mul_bwd: NULL pointer");
    XQ_REQUIRE(xq_aligned(gate, 16) && xq_aligned(up, 16) && xq_aligned(dh, 16) && xq_aligned(dgate, 16) && xq_aligned(dup, 16),
               "xq_silu_mul_bwd: pointers must be 16-byte aligned");
    silu_mul_bwd_kernel<<<dim3((unsigned)rows), 256, 0, (hipStream_t)stream>>>(
        (const bf16_t*)gate, (const bf16_t*)up, ld_in, (const bf16_t*)dh, ld_dh, row_w, (bf16_t*)dgate, (bf16_t*)dup,
        ld_out, d_row_w, rows, cols, limit);
    XQ_CHECK_LAUNCH("xq_silu_mul_bwd");
    return XQ_OK;
}
}  // namespace xq

extern "C" int xq_silu_mul_fwd(const void* gate, const void* up, int64_t ld_in, const float* row_w, void* h,
                               int64_t ld_h, int64_t rows, int64_t cols, void* stream) {
    return xq::silu_mul_fwd_limit(gate, up, ld_in, row_w, h, ld_h, rows, cols, 0.0f, stream);
}

extern "C" int xq_silu_mul_bwd(const void* gate, const void* up, int64_t ld_in, const void* dh, int64_t ld_dh,
                               const float* row_w, void* dgate, void* dup, int64_t ld_out, float* d_row_w,
                               int64_t rows, int64_t cols, void* stream) {
    return xq::silu_mul_bwd_limit(gate, up, ld_in, dh, ld_dh, row_w, dgate, dup, ld_out, d_row_w, rows, cols, 0.0f, stream);
}

extern "C" int64_t xq_route_workspace_bytes(int64_t n_routed, int32_t num_experts) {
    return xq_cdiv(n_routed > 0 ? n_routed : 1, RB_CHUNK) * (int64_t)num_experts * 4;
}

extern "C" int xq_route_build(const int32_t* selected, int64_t n_routed, int32_t num_experts, int32_t* counts,
                              int32_t* offsets, int32_t* scatter_index, int32_t* tile_offsets, void* workspace,
                              int64_t workspace_bytes, void* stream_) {
    XQ_REQUIRE(num_experts >= 1 && num_experts <= RB_MAX_E, "xq_route_build: num_experts %d out of range [1, %d]", num_experts, RB_MAX_E);
    XQ_REQUIRE(n_routed >= 0 && n_routed < (1ll << 31), "xq_route_build: bad n_routed");
    XQ_REQUIRE(counts && offsets && tile_offsets && (n_routed == 0 || (selected && scatter_index)), "xq_route_build: NULL pointer");
    XQ_REQUIRE(workspace && workspace_bytes >= xq_route_workspace_bytes(n_routed, num_experts), "xq_route_build: workspace too small");
    hipStream_t stream = (hipStream_t)stream_;
    int32_t n_chunks = (int32_t)xq_cdiv(n_routed > 0 ? n_routed : 1, RB_CHUNK);
    int32_t* cc = (int32_t*)workspace;
    route_hist_kernel<<<dim3(n_chunks), 64, 0, stream>>>(selected, n_routed, num_experts, cc);
    XQ_CHECK_LAUNCH("route_hist");
    static std::atomic<bool> scan_attr_set{false};   // the attribute call is idempotent: a race only repeats it
    if (!scan_attr_set) {
        if (hipFuncSetAttribute((const void*)route_scan_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 17 * RB_MAX_E * 4) != hipSuccess) {
            xq_set_error("xq_route_build: cannot raise the dynamic LDS limit");
            return XQ_ERR_LAUNCH;
        }
        scan_attr_set = true;
    }
    route_scan_kernel<<<dim3(1), 1024, (size_t)17 * num_experts * 4, stream>>>(cc, n_chunks, num_experts, counts, offsets, tile_offsets);
    XQ_CHECK_LAUNCH("route_scan");
    if (n_routed > 0) {
        int id_bits = 0;
        while ((1 << id_bits) < num_experts) ++id_bits;
        route_place_kernel<<<dim3(n_chunks), 64, 0, stream>>>(selected, n_routed, num_experts, id_bits, cc, offsets, scatter_index);
        XQ_CHECK_LAUNCH("route_place");
    }
    return XQ_OK;
}

extern "C" int xq_moe_scatter(const void* in, int64_t ld_in, const int32_t* scatter_index, int64_t n_routed,
                              int32_t topk, int64_t width, void* out, int64_t ld_out, void* stream) {
    XQ_REQUIRE(topk >= 1 && width % 8 == 0 && ld_in % 8 == 0 && ld_out % 8 == 0, "xq_moe_scatter: width/strides must be multiples of 8");
    if (n_routed == 0 || width == 0) return XQ_OK;
    XQ_REQUIRE(in && out && scatter_index && xq_aligned(in, 16) && xq_aligned(out, 16), "xq_moe_scatter: bad pointer");
    XQ_REQUIRE(n_routed % topk == 0, "xq_moe_scatter: n_routed %lld is not a multiple of topk %d", (long long)n_routed, topk);
    moe_scatter_kernel<<<dim3((unsigned)(n_routed / topk)), 256, 0, (hipStream_t)stream>>>((const bf16_t*)in, ld_in, scatter_index,
                                                                                           topk, width / 8, (bf16_t*)out, ld_out);
    XQ_CHECK_LAUNCH("xq_moe_scatter");
    return XQ_OK;
}

extern "C" int xq_moe_scatter_scalar(const void* src, int src_dtype, const int32_t* scatter_index, int64_t n, float* dst,
                                     void* stream) {
    if (n == 0) return XQ_OK;
    XQ_REQUIRE(src && dst && scatter_index, "xq_moe_scatter_scalar: NULL pointer");
    moe_scatter_scalar_kernel<<<dim3((unsigned)xq_cdiv(n, 256)), 256, 0, (hipStream_t)stream>>>(src, src_dtype == XQ_DT_F32,
                                                                                                scatter_index, n, dst);
    XQ_CHECK_LAUNCH("xq_moe_scatter_scalar");
    return XQ_OK;
}

extern "C" int xq_moe_gather_scalar(const float* src, const int32_t* scatter_index, int64_t n, void* dst, int dst_dtype,
                                    void* stream) {
    if (n == 0) return XQ_OK;
    XQ_REQUIRE(src && dst && scatter_index, "xq_moe_gather_scalar: NULL pointer");
    moe_gather_scalar_kernel<<<dim3((unsigned)xq_cdiv(n, 256)), 256, 0, (hipStream_t)stream>>>(src, scatter_index, n, dst,
                                                                                               dst_dtype == XQ_DT_F32);
    XQ_CHECK_LAUNCH("xq_moe_gather_scalar");
    return XQ_OK;
}

extern "C" int xq_moe_gather(const void* rows, const void* rows2, int64_t ld_rows, const int32_t* scatter_index,
                             int64_t n_tokens, int32_t topk, int64_t width, void* out, int64_t ld_out, void* stream) {
    XQ_REQUIRE(topk >= 1 && width % 8 == 0 && ld_rows % 8 == 0 && ld_out % 8 == 0, "xq_moe_gather: width/strides must be multiples of 8");
    if (n_tokens == 0 || width == 0) return XQ_OK;
    XQ_REQUIRE(rows && out && scatter_index && xq_aligned(rows, 16) && xq_aligned(out, 16) && (!rows2 || xq_aligned(rows2, 16)),
               "xq_moe_gather: bad pointer");
    if (rows2)
        moe_gather_kernel<true><<<dim3((unsigned)n_tokens), 256, 0, (hipStream_t)stream>>>(
            (const bf16_t*)rows, (const bf16_t*)rows2, ld_rows, scatter_index, topk, width / 8, (bf16_t*)out, ld_out);
    else
        moe_gather_kernel<false><<<dim3((unsigned)n_tokens), 256, 0, (hipStream_t)stream>>>(
            (const bf16_t*)rows, nullptr, ld_rows, scatter_index, topk, width / 8, (bf16_t*)out, ld_out);
    XQ_CHECK_LAUNCH("xq_moe_gather");
    return XQ_OK;
}
