// Host entry points of the fused dequant-GEMM + LoRA path (dense and grouped).
#include "xq_gemm_tile.h"
#include <algorithm>
#include <atomic>
#include "xq_gemm_256.h"
#include "xq_gemm_dtl.h"
#include <stdlib.h>
#include <mutex>
#include "xq_lora.h"
#include "xq_skinny.h"

namespace xq {

template <int FMT, int LAYOUT>
static void launch_tile_cc(const TileArgs& g, bool contract_cols, dim3 grid, hipStream_t s) {
    if (contract_cols) gemm_tile_kernel<FMT, LAYOUT, true><<<grid, 256, 0, s>>>(g);
    else gemm_tile_kernel<FMT, LAYOUT, false><<<grid, 256, 0, s>>>(g);
}

// kernel-selection policy (xq_set_tile_policy): 0 = by problem size, 1 = always the generic single-buffered
// tile kernel, 2 / 3 = the pipelined kernel with 256x256 / 128x128 tiles whenever the format allows it.
// XQ_SKINNY=0 disables the M <= 64 path.  Both are process-wide test switches: set them while no other thread is
// inside the library.
static int g_skinny_enabled = [] { const char* e = getenv("XQ_SKINNY"); return e ? atoi(e) : 1; }();
static int g_tile_policy = [] { const char* e = getenv("XQ_TILE_POLICY"); return e ? atoi(e) : 0; }();

template <typename K>
static int raise_lds_limit(K kernel, size_t bytes, const char* who) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) {
        xq_set_error("%s: cannot raise the dynamic LDS limit: %s", who, hipGetErrorString(e));
        return XQ_ERR_LAUNCH;
    }
    return XQ_OK;
}

template <int FMT, bool CC, bool GROUPED, int T, bool SPLIT256 = false>
static int launch_256_one(const G256Args& f, dim3 grid, hipStream_t s, const char* who) {
    static std::atomic<bool> attr_set{false};   // per instantiation; the attribute call is idempotent: a race only repeats it
    if (!attr_set) {
        int rc = raise_lds_limit(gemm_256_kernel<FMT, CC, GROUPED, T, SPLIT256>, Geo<T>::lds_bytes(CC), who);
        if (rc) return rc;
        attr_set = true;
    }
    gemm_256_kernel<FMT, CC, GROUPED, T, SPLIT256><<<grid, Geo<T>::NT, Geo<T>::lds_bytes(CC), s>>>(f);
    return XQ_OK;
}

// Block-fp8 launches on large unsplit tiles (dense and expert banks) run gemm_dtl16_kernel (1, the default) or gemm_256_kernel (0): a
// process-wide switch for tests and A/B measurements, XQ_FP8_DIRECT in the environment sets it at load time.
static std::atomic<int> g_fp8_direct{[] { const char* e = getenv("XQ_FP8_DIRECT"); return e ? atoi(e) : 1; }()};

static int launch_dtl16(const G256Args& f, bool cc, bool grouped, dim3 grid, hipStream_t s, const char* who) {
    static std::atomic<bool> attr_set{false};
    if (!attr_set) {
        int rc = raise_lds_limit(gemm_dtl16_kernel<true, 8, false>, GeoDtl::lds_total(), who);
        if (!rc) rc = raise_lds_limit(gemm_dtl16_kernel<false, 8, false>, GeoDtl::lds_total(), who);
        if (!rc) rc = raise_lds_limit(gemm_dtl16_kernel<true, 8, true>, GeoDtl::lds_total(), who);
        if (!rc) rc = raise_lds_limit(gemm_dtl16_kernel<false, 8, true>, GeoDtl::lds_total(), who);
        if (rc) return rc;
        attr_set = true;
    }
    if (grouped) {
        if (cc) gemm_dtl16_kernel<true, 8, true><<<grid, 512, GeoDtl::lds_total(), s>>>(f);
        else gemm_dtl16_kernel<false, 8, true><<<grid, 512, GeoDtl::lds_total(), s>>>(f);
    } else {
        if (cc) gemm_dtl16_kernel<true, 8, false><<<grid, 512, GeoDtl::lds_total(), s>>>(f);
        else gemm_dtl16_kernel<false, 8, false><<<grid, 512, GeoDtl::lds_total(), s>>>(f);
    }
    return XQ_OK;
}

template <int FMT, bool CC, bool GROUPED>
static int launch_256_t(const G256Args& f, int T, dim3 grid, hipStream_t s, const char* who) {
    if constexpr (!GROUPED)
        if (T == 256 && f.ksplit > 1) return launch_256_one<FMT, CC, false, 256, true>(f, grid, s, who);
    return T == 256 ? launch_256_one<FMT, CC, GROUPED, 256>(f, grid, s, who) : launch_256_one<FMT, CC, GROUPED, 128>(f, grid, s, who);
}

template <int FMT>
static int launch_256(const G256Args& f, bool cc, bool grouped, int T, dim3 grid, hipStream_t s, const char* who) {
    if (cc) return grouped ? launch_256_t<FMT, true, true>(f, T, grid, s, who) : launch_256_t<FMT, true, false>(f, T, grid, s, who);
    return grouped ? launch_256_t<FMT, false, true>(f, T, grid, s, who) : launch_256_t<FMT, false, false>(f, T, grid, s, who);
}

// compute units of the current device (256 on MI355X), asked once
int num_cus() {
    static std::atomic<int> cached{0};
    int c = cached.load(std::memory_order_relaxed);
    if (c > 0) return c;
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
        n = 256;
    cached.store(n, std::memory_order_relaxed);
    return n;
}

// Grid of the persistent program (large unsplit tiles): one block per compute unit, a multiple of 8 so that every
// tile of a block falls into the same XCD's range of the tile order; more blocks when a block would otherwise walk
// more tiles than it keeps a table for.  XQ_PERSIST=0 launches one block per tile (same kernel, same results).
static int g_persist = [] { const char* e = getenv("XQ_PERSIST"); return e ? atoi(e) : 1; }();
static inline unsigned persistent_grid(int64_t tiles) {
    if (!g_persist) return (unsigned)tiles;
    int64_t blocks = std::max<int64_t>((num_cus() / 8) * 8, 8);
    blocks = std::max(blocks, (xq_cdiv(tiles, G256_MAX_ROUNDS) + 7) / 8 * 8);
    return (unsigned)std::min(tiles, blocks);
}

// Tile size of a dense launch under the default policy: large tiles from the point where they fill more than
// half the chip (two small tiles are resident per compute unit, and finish sooner than a half-empty round of
// large ones).
static inline int dense_tile_size(int64_t n_rows, int64_t Nout) {
    return xq_cdiv(n_rows, 256) * xq_cdiv(Nout, 256) > num_cus() / 2 ? 256 : 128;
}

// K splits of a dense launch of `blocks` tiles of size T over nk K-steps (1 = none): used when the tiles fill at
// most half of the block slots of the chip (256 large tiles, 512 small ones); every split keeps at least 8 K-steps.
static inline int ksplit_for(int64_t blocks, int T, int64_t nk) {
    const int64_t slots = T == 256 ? num_cus() : 2 * num_cus();   // one large or two small tiles per compute unit
    if (blocks <= 0 || blocks * 2 > slots) return 1;
    int64_t s = slots / blocks;
    if (s > nk / 8) s = nk / 8;
    if (s > 8) s = 8;
    return s < 2 ? 1 : (int)s;
}

// How the default policy runs a dense [n_rows, Nout] product over nk K-steps: `head_rows` leading rows on tiles of
// size T in `split` K splits, and, when head_rows < n_rows, the trailing rows as a second launch.  A launch of large
// tiles whose last round would fill only part of the chip keeps the tile rows that make whole rounds and hands the
// others either to small tiles (two of those blocks share a CU) or to large tiles in K splits, whichever the
// estimates below make cheaper; the whole launch stays as it is unless that saves a fifth of a round.
struct DensePlan {
    int T, split;
    int64_t head_rows;
    int tail_T, tail_split;
};
static DensePlan plan_dense(int64_t n_rows, int64_t Nout, int64_t nk) {
    DensePlan p{dense_tile_size(n_rows, Nout), 1, n_rows, 0, 1};
    if (p.T == 128) {
        p.split = ksplit_for(xq_cdiv(n_rows, 128) * xq_cdiv(Nout, 128), 128, nk);
        return p;
    }
    const int64_t tr = xq_cdiv(n_rows, 256), tc = xq_cdiv(Nout, 256), cus = num_cus();
    const int64_t full = tr * tc / cus, rem = tr * tc - full * cus;
    const int64_t keep = full * cus / tc;                  // tile rows that stay on whole rounds of large tiles
    if (rem == 0 || keep == 0 || keep >= tr) return p;
    const int64_t tail_rows = n_rows - keep * 256;
    // costs in units of one round of large tiles (measured: small tiles take 0.54 of it with up to one block per
    // CU, 0.7 with up to two; a split large tile 1/S of it plus the pass over its fp32 partial sums at ~4 TB/s,
    // a round lasting ~1.9 us per K-step)
    const int64_t n128 = xq_cdiv(tail_rows, 128) * xq_cdiv(Nout, 128);
    const double small_cost = n128 <= cus ? 0.54 : 0.7 * (double)xq_cdiv(n128, 2 * cus);
    const int s256 = ksplit_for((tr - keep) * tc, 256, nk);
    const double round_us = 1.9 * (double)nk;
    const double split_cost = s256 > 1 ? 1.0 / s256 + (3.0 + (4.0 * s256 + 2.0) * (double)tail_rows * (double)Nout / 4.0e6) / round_us : 1e9;
    const double tail_cost = small_cost < split_cost ? small_cost : split_cost;
    if ((double)xq_cdiv(keep * tc, cus) + tail_cost < (double)(full + 1) - 0.2) {
        p.head_rows = keep * 256;
        if (split_cost < small_cost) { p.tail_T = 256; p.tail_split = s256; }
        else { p.tail_T = 128; p.tail_split = 1; }
    }
    return p;
}

// fp32 partial-sum bytes the split-K forms of a dense [n_rows, Nout] product over Kc may want, under any tile policy
int64_t tile_gemm_partial_bytes(int64_t n_rows, int64_t Nout, int64_t Kc) {
    if (n_rows <= 0 || Kc % BK) return 0;
    const int64_t nk = Kc / BK;
    int64_t elems = 0;
    for (int T : {128, 256}) {         // a whole launch on either tile size (default or forced policy)
        const int s = ksplit_for(xq_cdiv(n_rows, T) * xq_cdiv(Nout, T), T, nk);
        if (s > 1 && s * n_rows > elems) elems = s * n_rows;
    }
    const DensePlan p = plan_dense(n_rows, Nout, nk);
    if (p.head_rows < n_rows && p.tail_split > 1 && p.tail_split * (n_rows - p.head_rows) > elems)
        elems = p.tail_split * (n_rows - p.head_rows);
    return elems * Nout * 4;
}

// Whether a grouped launch on this bank may take a second bank of the same shape (see G256Args::W2): block-fp8 on the
// pipelined kernel, whole 256-column tiles per bank (which also keeps the K-step where the dgrad changes banks on a
// scale-block boundary and away from the pipeline's prologue).
bool two_banks_supported(const xq_weight* w) {
    return w->format == XQ_FMT_FP8 && g_tile_policy != 1 && w->cols % 256 == 0 && w->cols >= 512 && w->num_experts >= 1;
}

// Whether the dgrad of two dense [N, K] weights of one shape may run as one launch (see launch_tile_gemm): block-fp8 on
// the pipelined kernel, the change of matrix on a scale-block boundary and past the pipeline's prologue.
bool two_dense_supported(const xq_weight* w) {
    return w->format == XQ_FMT_FP8 && g_tile_policy != 1 && w->num_experts == 1 && w->rows % 128 == 0 && w->rows >= 512;
}

// C[rows, Nout] = A . op(deq(W)) (+ su . Lr^T) (+ bias); see xq_gemm_tile.h.  force_T = 256 / 128 fixes the tile
// size of the pipelined kernel (and force_split its K splits), 0 leaves both to the selection policy.  `partial` (may be NULL) is scratch for
// split-K sums; a launch that would split but finds less than tile_gemm_partial_bytes() there runs unsplit.
static int launch_tile_gemm_t(const xq_weight* w, bool contract_cols, const bf16_t* A, int64_t lda, int64_t n_rows,
                              const int32_t* offsets, const int32_t* tile_offsets, const bf16_t* su, const bf16_t* lora_right,
                              int r_pad, const bf16_t* bias, bf16_t* C, int64_t ldc, hipStream_t stream, const char* who,
                              int force_T, int force_split, float* partial, int64_t partial_bytes,
                              const TwoBanks* two = nullptr, const int32_t* a_rows = nullptr, int64_t a_span_rows = 0) {
    const int64_t a_rows_span = a_rows ? a_span_rows : n_rows;      // rows of A that the launch may touch (0: not known)
    TileArgs g;
    g.A = A; g.lda = lda; g.C = C; g.ldc = ldc;
    g.packed = (const uint8_t*)w->packed;
    g.scales = (const uint8_t*)w->scales;
    g.global_scale = w->global_scale;
    g.packed_stride = xq_packed_bytes_per_expert(w);
    g.scale_stride = xq_scale_bytes_per_expert(w);
    g.wrows = (int32_t)w->rows; g.wcols = (int32_t)w->cols;
    g.group = w->group; g.scale_dtype = w->scale_dtype;
    g.Kc = contract_cols ? g.wcols : g.wrows;
    g.Nout = contract_cols ? g.wrows : g.wcols;
    const bool two_dense = two && !offsets;
    if (two) {
        // a second matrix of the same shape.  Expert banks: twice the contraction (dgrad) or twice the output columns
        // (forward).  Dense [N, K] weights: the dgrad contracts over the rows of both, dX = [dY1 | dY2] . [W1 ; W2].
        XQ_REQUIRE(two->w2 && two->w2->rows == w->rows && two->w2->cols == w->cols && two->w2->num_experts == w->num_experts,
                   "%s: a two-matrix launch takes two weights of one shape", who);
        if (two_dense) {
            XQ_REQUIRE(!contract_cols && two_dense_supported(w) && two_dense_supported(two->w2),
                       "%s: the dense two-matrix form is the dgrad of two block-fp8 weights (out_features %% 128 == 0, >= 512)", who);
            g.Kc *= 2;
        } else {
            XQ_REQUIRE(two_banks_supported(w) && two_banks_supported(two->w2),
                       "%s: a two-bank launch takes two block-fp8 expert banks (columns a multiple of 256)", who);
            if (contract_cols) g.Kc *= 2;
            else g.Nout *= 2;
        }
    }
    g.n_rows = n_rows; g.offsets = offsets; g.tile_offsets = tile_offsets; g.num_experts = w->num_experts;
    g.su = su; g.lora_right = lora_right; g.r_pad = (su && lora_right) ? r_pad : 0;
    g.bias = bias;
    XQ_REQUIRE(g.Kc % BK == 0, "%s: contraction length %d must be a multiple of %d", who, g.Kc, BK);
    XQ_REQUIRE(g.Nout % 16 == 0, "%s: output width %d must be a multiple of 16", who, g.Nout);
    XQ_REQUIRE(lda % 8 == 0 && xq_aligned(A, 16), "%s: activation rows must be 16-byte aligned", who);
    XQ_REQUIRE(xq_aligned(w->packed, 16) && g.packed_stride % 16 == 0, "%s: packed weight must be 16-byte aligned", who);
    XQ_REQUIRE(g.r_pad == 0 || (g.r_pad % 16 == 0 && g.r_pad <= 64 && xq_aligned(su, 16) && xq_aligned(lora_right, 16)),
               "%s: bad low-rank side term (r_pad %d)", who, g.r_pad);
    if (w->format != XQ_FMT_FP8 && w->layout == XQ_LAYOUT_GKN)
        XQ_REQUIRE(w->rows % 2 == 0, "%s: GKN 4-bit storage needs an even row count", who);
    if (n_rows == 0) return XQ_OK;
    // block-fp8 and FLAT 4-bit weights: the pipelined tile kernel, 256x256 tiles when they fill the chip,
    // 128x128 tiles otherwise (dense or grouped)
    {
        const bool grouped = offsets != nullptr;
        int gshift = 0;
        while ((1 << gshift) < g.group) ++gshift;
        // 4-bit: power-of-two groups of at least 16; dense matrices FLAT, expert banks GKN (16-byte pieces of codes
        // and of scales: columns in multiples of 16, 16-byte aligned scale storage)
        const bool fmt_ok = w->format == XQ_FMT_FP8 ||
                            ((1 << gshift) == g.group && g.group >= 16 &&
                             (grouped ? w->layout == XQ_LAYOUT_GKN && g.wcols % 16 == 0 && g.wrows >= 2 &&
                                            xq_aligned(w->scales, 16) && g.scale_stride % 16 == 0
                                      : w->layout == XQ_LAYOUT_FLAT));
        const bool big = grouped && n_rows >= 128ll * w->num_experts && n_rows >= 8192;   // grouped: large tiles
        const DensePlan plan = plan_dense(n_rows, g.Nout, g.Kc / BK);
        const bool planned = !grouped && fmt_ok && g_tile_policy == 0 && force_T == 0 && !two_dense;   // two matrices: one unsplit launch
        const int T = force_T ? force_T : g_tile_policy == 2 ? 256 : g_tile_policy == 3 ? 128 : grouped ? (big ? 256 : 128) : plan.T;
        if (planned && plan.head_rows < n_rows) {
            const int64_t head = plan.head_rows;
            const int rc = launch_tile_gemm_t(w, contract_cols, A, lda, head, nullptr, nullptr, su, lora_right, r_pad,
                                              bias, C, ldc, stream, who, 256, 1, nullptr, 0);
            if (rc) return rc;
            return launch_tile_gemm_t(w, contract_cols, A + head * lda, lda, n_rows - head, nullptr, nullptr,
                                      su ? su + head * r_pad : nullptr, lora_right, r_pad, bias, C + head * ldc, ldc,
                                      stream, who, plan.tail_T, plan.tail_split, partial, partial_bytes);
        }
        const int64_t tiles_m = xq_cdiv(n_rows, T) + (grouped ? w->num_experts : 0);
        const int64_t tiles_n = xq_cdiv(g.Nout, T);
        if (fmt_ok && g_tile_policy != 1 && tiles_m * tiles_n < (1ll << 31)) {
            G256Args f;
            f.A = A; f.lda = lda; f.a_rows = a_rows; f.C = C; f.ldc = ldc;
            f.W = g.packed; f.scales = g.scales; f.global_scale = g.global_scale;
            f.packed_stride = g.packed_stride; f.scale_stride = g.scale_stride;
            f.wrows = g.wrows; f.wcols = g.wcols; f.gshift = gshift; f.scale_dtype = g.scale_dtype;
            f.Kc = g.Kc; f.Nout = g.Nout; f.M = n_rows;
            f.offsets = offsets;
            f.tile_prefix = !grouped ? nullptr : (T == 256 ? tile_offsets + (w->num_experts + 1) : tile_offsets);
            f.num_experts = w->num_experts;
            f.su = g.r_pad ? su : nullptr; f.lora_right = g.r_pad ? lora_right : nullptr; f.r_pad = g.r_pad;
            f.bias = bias;
            f.tiles_m = (int32_t)tiles_m; f.tiles_n = (int32_t)tiles_n;
            int ksplit = grouped || two_dense ? 1 : force_T ? force_split : planned ? plan.split : ksplit_for(tiles_m * tiles_n, T, g.Kc / BK);
            if (ksplit > 1 && (!partial || !xq_aligned(partial, 16) || partial_bytes < (int64_t)ksplit * n_rows * g.Nout * 4)) ksplit = 1;
            f.ksplit = ksplit; f.partial = ksplit > 1 ? partial : nullptr;
            f.W2 = nullptr; f.scales2 = nullptr; f.su2 = nullptr; f.lora_right2 = nullptr; f.ncols1 = 0; f.nk1 = 0;
            f.ld_su = g.r_pad; f.H = nullptr; f.ldh = 0; f.bias2 = nullptr;
            f.wide_rows = xq_aligned(C, 16) && ldc % 8 == 0 && xq_aligned(bias, 8);
            if (two) {
                f.W2 = (const uint8_t*)two->w2->packed; f.scales2 = (const uint8_t*)two->w2->scales;
                f.su2 = g.r_pad ? two->su2 : nullptr; f.lora_right2 = g.r_pad ? two->lora_right2 : nullptr;
                f.ncols1 = g.wcols; f.nk1 = (two_dense ? g.wrows : g.wcols) / BK;
            }
            // (the kernel's own rule: large unsplit tiles, except the 4-bit expert banks)
            const bool persistent = T == 256 && ksplit == 1 && !(grouped && w->format != XQ_FMT_FP8);
            dim3 grid(persistent ? persistent_grid(tiles_m * tiles_n) : (unsigned)(tiles_m * tiles_n), (unsigned)ksplit);
            const bool timed = xq_profile_mark_begin(stream, 2.0 * (double)n_rows * g.Nout * ((double)g.Kc + g.r_pad));
            int rc;
            // block-fp8 on large unsplit tiles, dense or expert banks: the kernel that brings both operand tiles straight into LDS
            // and decodes after the fragment read (xq_gemm_dtl.h), one block per tile
            const int nk_all = g.Kc / BK;
            // (two matrices: the second one starts on a scale-block boundary of the contraction, or -- two banks side by side
            // in a forward -- on a tile boundary of the columns)
            const bool two_ok = !two || ((grouped && !contract_cols) ? f.ncols1 % 256 == 0 : (f.nk1 % 2 == 0 && f.nk1 >= 2));
            if (g_fp8_direct && w->format == XQ_FMT_FP8 && T == 256 && ksplit == 1 && nk_all >= 3 &&
                nk_all <= 2 * GeoDtl::SCL_MAX && two_ok && (!grouped || g.wcols % 16 == 0) &&
                // (its lanes address their operands by 32-bit byte offsets from a base)
                a_rows_span > 0 && a_rows_span * lda * 2 < (1ll << 32) && (int64_t)g.wrows * g.wcols < (1ll << 32))
                rc = launch_dtl16(f, contract_cols, grouped, dim3((unsigned)(tiles_m * tiles_n)), stream, who);
            else if (w->format == XQ_FMT_FP8) rc = launch_256<XQ_FMT_FP8>(f, contract_cols, grouped, T, grid, stream, who);
            else if (w->format == XQ_FMT_INT4) rc = launch_256<XQ_FMT_INT4>(f, contract_cols, grouped, T, grid, stream, who);
            else if (w->format == XQ_FMT_NF4) rc = launch_256<XQ_FMT_NF4>(f, contract_cols, grouped, T, grid, stream, who);
            else rc = launch_256<XQ_FMT_NVFP4>(f, contract_cols, grouped, T, grid, stream, who);
            if (rc) return rc;
            XQ_CHECK_LAUNCH(who);
            if (ksplit > 1) {
                const int64_t quads = n_rows * (g.Nout >> 2);
                splitk_reduce_kernel<<<(unsigned)xq_cdiv(quads, 256), 256, 0, stream>>>(partial, ksplit, n_rows, g.Nout, C, ldc);
                XQ_CHECK_LAUNCH(who);
            }
            if (timed) xq_profile_mark_end(stream);
            return XQ_OK;
        }
    }
    XQ_REQUIRE(!a_rows, "%s: internal error: a row map needs the pipelined tile kernel (see tile_gemm_takes_row_map)", who);
    unsigned mt = (unsigned)(xq_cdiv(n_rows, BM) + (offsets ? w->num_experts : 0));
    dim3 grid(mt, (unsigned)xq_cdiv(g.Nout, BN));
    const bool timed = xq_profile_mark_begin(stream, 2.0 * (double)n_rows * g.Nout * ((double)g.Kc + g.r_pad));
    if (w->format == XQ_FMT_FP8) launch_tile_cc<XQ_FMT_FP8, XQ_LAYOUT_FLAT>(g, contract_cols, grid, stream);
    else if (w->format == XQ_FMT_INT4 && w->layout == XQ_LAYOUT_FLAT) launch_tile_cc<XQ_FMT_INT4, XQ_LAYOUT_FLAT>(g, contract_cols, grid, stream);
    else if (w->format == XQ_FMT_INT4) launch_tile_cc<XQ_FMT_INT4, XQ_LAYOUT_GKN>(g, contract_cols, grid, stream);
    else if (w->format == XQ_FMT_NF4 && w->layout == XQ_LAYOUT_FLAT) launch_tile_cc<XQ_FMT_NF4, XQ_LAYOUT_FLAT>(g, contract_cols, grid, stream);
    else if (w->format == XQ_FMT_NF4) launch_tile_cc<XQ_FMT_NF4, XQ_LAYOUT_GKN>(g, contract_cols, grid, stream);
    else if (w->layout == XQ_LAYOUT_FLAT) launch_tile_cc<XQ_FMT_NVFP4, XQ_LAYOUT_FLAT>(g, contract_cols, grid, stream);
    else launch_tile_cc<XQ_FMT_NVFP4, XQ_LAYOUT_GKN>(g, contract_cols, grid, stream);
    if (timed) xq_profile_mark_end(stream);
    XQ_CHECK_LAUNCH(who);
    return XQ_OK;
}

// gate | up | SwiGLU of a dense block-fp8 MLP in one launch: gu[M, 2I] = (x . deq(Wg)^T + side term | x . deq(Wu)^T +
// side term) and h[M, I] = bf16(silu(gate)) * up from the rounded projections.  Both weights [I, K] block-fp8.
int launch_gate_up_swiglu(const xq_weight* wg, const xq_weight* wu, const bf16_t* x, int64_t ldx, int64_t M,
                          const bf16_t* su_g, const bf16_t* su_u, int64_t ld_su, const bf16_t* lr_g, const bf16_t* lr_u,
                          int r_pad, const bf16_t* bias_g, const bf16_t* bias_u, bf16_t* gu, int64_t ldgu, bf16_t* h,
                          int64_t ldh, hipStream_t stream) {
    static const char* who = "gate_up_swiglu";
    XQ_REQUIRE(wg->format == XQ_FMT_FP8 && wu->format == XQ_FMT_FP8 && wg->rows == wu->rows && wg->cols == wu->cols,
               "%s: two block-fp8 weights of one shape", who);
    const int64_t I = wg->rows, K = wg->cols;
    XQ_REQUIRE(K % BK == 0 && I % 16 == 0, "%s: in_features %% 64 == 0 and out_features %% 16 == 0", who);
    XQ_REQUIRE(ldx % 8 == 0 && xq_aligned(x, 16) && xq_aligned(wg->packed, 16) && xq_aligned(wu->packed, 16),
               "%s: operands must be 16-byte aligned", who);
    XQ_REQUIRE(ldgu % 8 == 0 && ldh % 8 == 0 && xq_aligned(gu, 16) && xq_aligned(h, 16), "%s: output rows must be 16-byte aligned", who);
    XQ_REQUIRE(xq_aligned(bias_g, 8) && xq_aligned(bias_u, 8), "%s: bias vectors must be 8-byte aligned", who);
    const bool side = su_g && su_u && lr_g && lr_u && r_pad > 0;
    XQ_REQUIRE(!side || (r_pad % 16 == 0 && r_pad <= 64 && ld_su >= r_pad && ld_su % 8 == 0 && xq_aligned(su_g, 16) &&
                         xq_aligned(su_u, 16) && xq_aligned(lr_g, 16) && xq_aligned(lr_u, 16)),
               "%s: bad low-rank side term", who);
    if (M == 0) return XQ_OK;
    G256Args f{};
    f.A = x; f.lda = ldx; f.C = gu; f.ldc = ldgu;
    f.W = (const uint8_t*)wg->packed; f.scales = (const uint8_t*)wg->scales;
    f.W2 = (const uint8_t*)wu->packed; f.scales2 = (const uint8_t*)wu->scales;
    f.wrows = (int32_t)I; f.wcols = (int32_t)K; f.scale_dtype = XQ_SCALE_F32;
    f.Kc = (int32_t)K; f.Nout = (int32_t)I; f.M = M;
    f.num_experts = 1;
    f.su = side ? su_g : nullptr; f.su2 = side ? su_u : nullptr; f.ld_su = ld_su;
    f.lora_right = side ? lr_g : nullptr; f.lora_right2 = side ? lr_u : nullptr; f.r_pad = side ? r_pad : 0;
    f.bias = bias_g; f.bias2 = bias_u;
    f.tiles_m = (int32_t)xq_cdiv(M, 256); f.tiles_n = (int32_t)xq_cdiv(I, 128);
    f.ksplit = 1;
    f.H = h; f.ldh = ldh;
    f.wide_rows = 1;
    static std::atomic<bool> attr_set{false};
    if (!attr_set) {
        int rc = raise_lds_limit(gemm_256_kernel<XQ_FMT_FP8, true, false, 256, false, true>, Geo<256>::lds_bytes(true), who);
        if (rc) return rc;
        attr_set = true;
    }
    // flops of the two projections and their side terms
    const bool timed = xq_profile_mark_begin(stream, 2.0 * (double)M * (2.0 * I) * ((double)K + f.r_pad));
    gemm_256_kernel<XQ_FMT_FP8, true, false, 256, false, true>
        <<<dim3(persistent_grid((int64_t)f.tiles_m * f.tiles_n)), Geo<256>::NT, Geo<256>::lds_bytes(true), stream>>>(f);
    XQ_CHECK_LAUNCH(who);
    if (timed) xq_profile_mark_end(stream);
    return XQ_OK;
}

int launch_tile_gemm(const xq_weight* w, bool contract_cols, const bf16_t* A, int64_t lda, int64_t n_rows,
                     const int32_t* offsets, const int32_t* tile_offsets, const bf16_t* su, const bf16_t* lora_right,
                     int r_pad, const bf16_t* bias, bf16_t* C, int64_t ldc, hipStream_t stream, const char* who,
                     float* partial, int64_t partial_bytes, const TwoBanks* two, const int32_t* a_rows, int64_t a_span_rows) {
    XQ_REQUIRE(!a_rows || offsets, "%s: a row map goes with a grouped launch", who);
    return launch_tile_gemm_t(w, contract_cols, A, lda, n_rows, offsets, tile_offsets, su, lora_right, r_pad, bias, C, ldc,
                              stream, who, 0, 1, partial, partial_bytes, two, a_rows, a_span_rows);
}

// whether a grouped launch over this bank runs on the pipelined tile kernel, which can read its activation rows through
// a row map (the conditions of launch_tile_gemm_t)
bool tile_gemm_takes_row_map(const xq_weight* w) {
    if (g_tile_policy == 1) return false;
    if (w->format == XQ_FMT_FP8) return true;
    int gshift = 0;
    while ((1 << gshift) < w->group) ++gshift;
    return (1 << gshift) == w->group && w->group >= 16 && w->layout == XQ_LAYOUT_GKN && w->cols % 16 == 0 && w->rows >= 2 &&
           xq_aligned(w->scales, 16) && xq_scale_bytes_per_expert(w) % 16 == 0;
}

static inline int64_t align256(int64_t b) { return (b + 255) & ~(int64_t)255; }
static inline int r_pad_of(int r) { return r <= 0 ? 0 : ((r + 15) / 16) * 16; }

struct Carver {
    uint8_t* base;
    int64_t used, cap;
    void* take(int64_t bytes) {
        void* p = base ? base + used : nullptr;
        used += align256(bytes);
        return p;
    }
};

}  // namespace xq

using namespace xq;

extern "C" int xq_set_tile_policy(int policy) {
    XQ_REQUIRE(policy >= 0 && policy <= 3, "xq_set_tile_policy: policy %d not in {0, 1, 2, 3}", policy);
    g_tile_policy = policy;
    return XQ_OK;
}

extern "C" int xq_set_skinny_one_launch(int enabled) {
    set_skinny_rows(enabled ? 1 : 0);
    return XQ_OK;
}

extern "C" int xq_set_skinny_gemv(int enabled) {
    set_skinny_gemv(enabled);
    return XQ_OK;
}

extern "C" int xq_set_skinny_spin_limit(int limit) {
    set_skinny_rows_spin_limit(limit);
    return XQ_OK;
}

extern "C" int xq_skinny_reset(void) { return reset_skinny_rows_slots(); }

extern "C" int xq_skinny_status(int* gave_up, int* failed_slots, void* stream) {
    int a = 0, b = 0;
    const int rc = skinny_rows_status(&a, &b, (hipStream_t)stream);
    if (gave_up) *gave_up = a;
    if (failed_slots) *failed_slots = b;
    return rc;
}

extern "C" int xq_set_fp8_direct_tiles(int enabled) {
    g_fp8_direct = enabled != 0;
    return XQ_OK;
}

extern "C" int xq_set_persistent_tiles(int enabled) {
    g_persist = enabled != 0;
    return XQ_OK;
}

extern "C" int64_t xq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int r) {
    int rp = r_pad_of(r);
    int64_t skinny = M <= 64 ? skinny_workspace_bytes(M, N, K, rp) : 0;
    // split-K partial sums of the forward (output N, contraction K) and of the dgrad (output K, contraction N)
    const int64_t pf = align256(tile_gemm_partial_bytes(M, N, K));
    const int64_t pb = align256(tile_gemm_partial_bytes(M, K, N));
    int64_t need = (pf > pb ? pf : pb) + 256;
    if (rp) {
        int64_t fwd = align256(rp * K * 2) + align256(N * rp * 2) + align256(M * rp * 2) + pf;
        int64_t tnp = tn_partial_bytes(M, N, rp);
        int64_t tnk = tn_partial_bytes(M, K, rp);
        int64_t tn = align256(tnp > tnk ? tnp : tnk);     // the weight-gradient partials reuse the dgrad's region
        int64_t bwd = align256(rp * N * 2) + align256(K * rp * 2) + align256(rp * K * 2) + 2 * align256(M * rp * 2) +
                      (tn > pb ? tn : pb);
        need = (fwd > bwd ? fwd : bwd) + 256;
    }
    return need > skinny ? need : skinny;
}

static int check_dense(const xq_weight* w, const char* who) {
    int rc = xq_validate_weight(w, who);
    if (rc) return rc;
    XQ_REQUIRE(w->num_experts == 1, "%s: dense entry point takes a single matrix", who);
    XQ_REQUIRE(w->format == XQ_FMT_FP8 || w->layout == XQ_LAYOUT_FLAT, "%s: dense weights are FLAT [N, K]", who);
    return XQ_OK;
}

extern "C" int xq_linear_fwd(const xq_weight* w, const void* x, int64_t ldx, int64_t M, const void* lora_A,
                             const void* lora_B, int lora_dtype, int r, float scaling, const void* bias_bf16, void* y,
                             int64_t ldy, void* su_out, void* workspace, int64_t workspace_bytes, void* stream_) {
    int rc = check_dense(w, "xq_linear_fwd");
    if (rc) return rc;
    const int64_t N = w->rows, K = w->cols;
    XQ_REQUIRE(M >= 0 && (M == 0 || (x && y)), "xq_linear_fwd: NULL activation pointer");   // an empty batch has no storage
    XQ_REQUIRE(r >= 0 && r <= 64, "xq_linear_fwd: LoRA rank %d out of range [0, 64]", r);
    XQ_REQUIRE(r == 0 || (lora_A && lora_B), "xq_linear_fwd: LoRA factors are NULL");
    XQ_REQUIRE(lora_dtype == XQ_DT_F32 || lora_dtype == XQ_DT_BF16, "xq_linear_fwd: bad lora_dtype");
    hipStream_t stream = (hipStream_t)stream_;
    if (M == 0) return XQ_OK;
    XQ_REQUIRE(ldy % 8 == 0 && xq_aligned(y, 16), "xq_linear_fwd: y rows must be 16-byte aligned");
    const int rp = r_pad_of(r);
    // decode / rollout shapes: stream the packed weight once (HBM-bound kernel); forward only
    if (!su_out && g_skinny_enabled && skinny_supported(w, M))
        return launch_skinny(w, (const bf16_t*)x, ldx, M, lora_A, lora_B, lora_dtype, r, scaling,
                             (const bf16_t*)bias_bf16, (bf16_t*)y, ldy, workspace, workspace_bytes, stream);
    bf16_t *A_bf = nullptr, *Bl = nullptr, *su = nullptr;
    Carver cv{(workspace && xq_aligned(workspace, 256)) ? (uint8_t*)workspace : nullptr, 0, workspace_bytes};
    if (rp) {
        XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= xq_linear_workspace_bytes(M, N, K, r),
                   "xq_linear_fwd: workspace missing, misaligned or smaller than xq_linear_workspace_bytes()");
        A_bf = (bf16_t*)cv.take(rp * K * 2);
        Bl = (bf16_t*)cv.take(N * rp * 2);
        su = su_out ? (bf16_t*)su_out : (bf16_t*)cv.take(M * rp * 2);
        FactorPrepJobs jobs{};
        jobs.in_f32 = lora_dtype == XQ_DT_F32;
        jobs.add(lora_A, r, K, false, A_bf, rp, K);
        jobs.add(lora_B, N, r, false, Bl, N, rp);
        if ((rc = launch_factor_prep_multi(jobs, stream))) return rc;
        if ((rc = launch_small_nt((const bf16_t*)x, ldx, M, K, A_bf, rp, scaling, su, nullptr, nullptr, 1, true, stream))) return rc;
    }
    // what is left of the workspace holds split-K partial sums (small row counts); without it the launch is unsplit
    float* partial = (float*)cv.take(0);
    return launch_tile_gemm(w, true, (const bf16_t*)x, ldx, M, nullptr, nullptr, su, Bl, rp, (const bf16_t*)bias_bf16,
                            (bf16_t*)y, ldy, stream, "xq_linear_fwd", partial, partial ? workspace_bytes - cv.used : 0);
}

// ---- forward for callers that cannot allocate ------------------------------------------------------------------
// The scratch of xq_linear_fwd (prepared LoRA panels, the [M, r_pad] intermediate, split-K partial sums) in an
// array that is part of the loaded code object: each device the library runs on holds its own copy at its own
// address until the process ends.  Host code reaches it only through the address hipGetSymbolAddress returns with
// that device current; the array's name is a host-side handle, never a device address.
static __device__ __align__(256) unsigned char scratch[XQ_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};
}  // namespace

// device address of this device's copy of `scratch` (resolved once per device, with that device current)
static int static_scratch(void** out, const char* who) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        xq_set_error("%s: cannot identify the current device: %s", who, hipGetErrorString(e));
        return XQ_ERR_LAUNCH;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            xq_set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return XQ_OK;
}

extern "C" int64_t xq_static_scratch_bytes(void) { return XQ_STATIC_SCRATCH_BYTES; }

extern "C" int64_t xq_linear_fwd_swiglu_workspace_bytes(int64_t M, int64_t N2, int64_t K, int r) {
    if (M < 0 || N2 < 0) return 0;
    return align256(xq_linear_workspace_bytes(M, N2, K, r)) + align256(M * N2 * 2) + 256;
}

extern "C" int xq_linear_fwd_swiglu(const xq_weight* w, const void* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                                    int lora_dtype, int r, float scaling, const void* bias_bf16, void* h, int64_t ldh, void* workspace,
                                    int64_t workspace_bytes, void* stream_) {
    int rc = check_dense(w, "xq_linear_fwd_swiglu");
    if (rc) return rc;
    const int64_t N2 = w->rows, K = w->cols, I = N2 / 2;
    XQ_REQUIRE(N2 % 16 == 0, "xq_linear_fwd_swiglu: the weight holds gate | up, [2 I, K] with I %% 8 == 0; got %lld rows", (long long)N2);
    XQ_REQUIRE(M >= 0 && (M == 0 || (x && h)), "xq_linear_fwd_swiglu: NULL activation pointer");
    XQ_REQUIRE(r >= 0 && r <= 64, "xq_linear_fwd_swiglu: LoRA rank %d out of range [0, 64]", r);
    XQ_REQUIRE(r == 0 || (lora_A && lora_B), "xq_linear_fwd_swiglu: LoRA factors are NULL");
    XQ_REQUIRE(lora_dtype == XQ_DT_F32 || lora_dtype == XQ_DT_BF16, "xq_linear_fwd_swiglu: bad lora_dtype");
    if (M == 0) return XQ_OK;
    XQ_REQUIRE(ldh % 8 == 0 && xq_aligned(h, 16), "xq_linear_fwd_swiglu: h rows must be 16-byte aligned");
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= xq_linear_fwd_swiglu_workspace_bytes(M, N2, K, r),
               "xq_linear_fwd_swiglu: workspace missing, misaligned or smaller than xq_linear_fwd_swiglu_workspace_bytes()");
    hipStream_t stream = (hipStream_t)stream_;
    // decode sizes: one launch that holds a column's gate and up rows in the same block
    if (g_skinny_enabled && skinny_rows_enabled() && skinny_supported(w, M) && ldx % 8 == 0 && ldx < (1ll << 31) && xq_aligned(x, 16) &&
        xq_aligned(w->packed, 16) && skinny_rows_swiglu_supported(w, M, lora_A, lora_B, lora_dtype, r)) {
        const double bytes = (double)xq_packed_bytes_per_expert(w) + (double)xq_scale_bytes_per_expert(w) + 2.0 * M * K + 2.0 * M * I +
                             4.0 * r * (K + N2);
        const bool timed = xq_profile_mark_begin(stream, bytes);
        rc = launch_skinny_rows_swiglu(w, (const bf16_t*)x, ldx, M, lora_A, lora_B, r, scaling, (const bf16_t*)bias_bf16, (bf16_t*)h, ldh,
                                       workspace, stream);
        if (rc != XQ_ERR_UNSUPPORTED) {      // (unsupported: no slot for the low-rank exchange could be had; nothing was launched)
            if (timed) xq_profile_mark_end(stream);
            if (rc) return rc;
            XQ_CHECK_LAUNCH("skinny forward with SwiGLU");
            return XQ_OK;
        }
    }
    // otherwise the forward into the workspace, then the elementwise kernel
    const int64_t lin = align256(xq_linear_workspace_bytes(M, N2, K, r));
    bf16_t* gu = (bf16_t*)((uint8_t*)workspace + lin);
    if ((rc = xq_linear_fwd(w, x, ldx, M, lora_A, lora_B, lora_dtype, r, scaling, bias_bf16, gu, N2, nullptr, workspace, lin, stream_))) return rc;
    return xq_silu_mul_fwd(gu, gu + I, N2, nullptr, h, ldh, M, I, stream_);
}

extern "C" int64_t xq_linear_fwd_multi_workspace_bytes(const xq_linear_job* jobs, int n_jobs, int64_t M) {
    int64_t need = 256 * 8;
    if (!jobs) return need;
    for (int i = 0; i < n_jobs; ++i) {
        if (!jobs[i].w) continue;
        const int64_t b = xq_linear_workspace_bytes(M, jobs[i].w->rows, jobs[i].w->cols, jobs[i].r);
        if (b > need) need = b;
    }
    return need;
}

extern "C" int xq_linear_fwd_multi(const xq_linear_job* jobs, int n_jobs, const void* x, int64_t ldx, int64_t M, int lora_dtype,
                                   void* workspace, int64_t workspace_bytes, void* stream_) {
    XQ_REQUIRE(jobs && n_jobs >= 1 && n_jobs <= XQ_LINEAR_MULTI_MAX, "xq_linear_fwd_multi: %d forwards (1 .. %d are taken)", n_jobs,
               XQ_LINEAR_MULTI_MAX);
    XQ_REQUIRE(lora_dtype == XQ_DT_F32 || lora_dtype == XQ_DT_BF16, "xq_linear_fwd_multi: bad lora_dtype");
    for (int i = 0; i < n_jobs; ++i) {
        XQ_REQUIRE(jobs[i].w, "xq_linear_fwd_multi: forward %d has no weight", i);
        int rc = check_dense(jobs[i].w, "xq_linear_fwd_multi");
        if (rc) return rc;
        XQ_REQUIRE(jobs[i].w->cols == jobs[0].w->cols, "xq_linear_fwd_multi: forward %d contracts over %lld features, forward 0 over %lld", i,
                   (long long)jobs[i].w->cols, (long long)jobs[0].w->cols);
        XQ_REQUIRE(jobs[i].r >= 0 && jobs[i].r <= 64, "xq_linear_fwd_multi: LoRA rank %d out of range [0, 64]", jobs[i].r);
        XQ_REQUIRE(jobs[i].r == 0 || (jobs[i].lora_A && jobs[i].lora_B), "xq_linear_fwd_multi: LoRA factors are NULL");
        XQ_REQUIRE(M == 0 || jobs[i].y, "xq_linear_fwd_multi: NULL output pointer");
        XQ_REQUIRE(M == 0 || (jobs[i].ldy % 8 == 0 && xq_aligned(jobs[i].y, 16)), "xq_linear_fwd_multi: y rows must be 16-byte aligned");
    }
    XQ_REQUIRE(M >= 0 && (M == 0 || x), "xq_linear_fwd_multi: NULL activation pointer");
    if (M == 0) return XQ_OK;
    hipStream_t stream = (hipStream_t)stream_;
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= xq_linear_fwd_multi_workspace_bytes(jobs, n_jobs, M),
               "xq_linear_fwd_multi: workspace missing, misaligned or smaller than xq_linear_fwd_multi_workspace_bytes()");
    // decode shapes that fit the whole-row kernel: every forward in one launch
    if (g_skinny_enabled && skinny_rows_enabled() && n_jobs > 1 && ldx % 8 == 0 && xq_aligned(x, 16)) {
        SkinnyRowsJob rj[XQ_LINEAR_MULTI_MAX];
        double bytes = 2.0 * M * jobs[0].w->cols;
        bool ok = true;
        for (int i = 0; i < n_jobs; ++i) {
            const xq_weight* w = jobs[i].w;
            rj[i] = SkinnyRowsJob{w, jobs[i].lora_A, jobs[i].lora_B, jobs[i].r, jobs[i].scaling, (const bf16_t*)jobs[i].bias_bf16,
                                  (bf16_t*)jobs[i].y, jobs[i].ldy};
            ok = ok && skinny_supported(w, M) && xq_aligned(w->packed, 16);
            bytes += (double)xq_packed_bytes_per_expert(w) + (double)xq_scale_bytes_per_expert(w) + 2.0 * M * w->rows +
                     4.0 * jobs[i].r * (w->cols + w->rows);
        }
        if (ok && skinny_rows_multi_supported(rj, n_jobs, M, lora_dtype)) {
            const bool timed = xq_profile_mark_begin(stream, bytes);
            const int rc = launch_skinny_rows_multi(rj, n_jobs, (const bf16_t*)x, ldx, M, workspace, stream);
            if (rc != XQ_ERR_UNSUPPORTED) {  // (unsupported: no slots for the low-rank exchange could be had; nothing was launched)
                if (timed) xq_profile_mark_end(stream);
                if (rc) return rc;
                XQ_CHECK_LAUNCH("skinny forwards");
                return XQ_OK;
            }
        }
    }
    // otherwise one after the other (the workspace is reused: the launches are ordered by the stream)
    for (int i = 0; i < n_jobs; ++i) {
        const int rc = xq_linear_fwd(jobs[i].w, x, ldx, M, jobs[i].lora_A, jobs[i].lora_B, lora_dtype, jobs[i].r, jobs[i].scaling,
                                     jobs[i].bias_bf16, jobs[i].y, jobs[i].ldy, nullptr, workspace, workspace_bytes, stream_);
        if (rc) return rc;
    }
    return XQ_OK;
}

extern "C" int xq_linear_fwd_static(const xq_weight* w, const void* x, int64_t ldx, int64_t M, const void* lora_A,
                                    const void* lora_B, int lora_dtype, int r, float scaling, const void* bias_bf16,
                                    void* y, int64_t ldy, void* stream_) {
    int rc = check_dense(w, "xq_linear_fwd_static");
    if (rc) return rc;
    XQ_REQUIRE(M >= 0, "xq_linear_fwd_static: negative row count");
    XQ_REQUIRE(r >= 0 && r <= 64, "xq_linear_fwd_static: LoRA rank %d out of range [0, 64]", r);
    const int64_t need = xq_linear_workspace_bytes(M, w->rows, w->cols, r);
    XQ_REQUIRE(need <= XQ_STATIC_SCRATCH_BYTES,
               "xq_linear_fwd_static: M=%lld, N=%lld, K=%lld, r=%d needs %lld bytes of scratch, the built-in buffer "
               "holds %lld; use xq_linear_fwd with a caller workspace",
               (long long)M, (long long)w->rows, (long long)w->cols, r, (long long)need,
               (long long)XQ_STATIC_SCRATCH_BYTES);
    void* ws = nullptr;
    if ((rc = static_scratch(&ws, "xq_linear_fwd_static"))) return rc;
    // nothing in the forward reads scratch it has not written in the same call (no counters, no accumulation into
    // memory), so the previous call's contents need no clearing
    return xq_linear_fwd(w, x, ldx, M, lora_A, lora_B, lora_dtype, r, scaling, bias_bf16, y, ldy, nullptr, ws,
                         XQ_STATIC_SCRATCH_BYTES, stream_);
}

extern "C" int xq_linear_bwd(const xq_weight* w, const void* x, int64_t ldx, const void* dy, int64_t lddy, int64_t M,
                             const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                             const void* su_in, void* dx, int64_t lddx, float* dA, float* dB, void* workspace,
                             int64_t workspace_bytes, void* stream_) {
    int rc = check_dense(w, "xq_linear_bwd");
    if (rc) return rc;
    const int64_t N = w->rows, K = w->cols;
    XQ_REQUIRE(M >= 0 && (M == 0 || dy), "xq_linear_bwd: dy is NULL");
    XQ_REQUIRE(r >= 0 && r <= 64, "xq_linear_bwd: LoRA rank %d out of range [0, 64]", r);
    XQ_REQUIRE(r == 0 || (lora_A && lora_B), "xq_linear_bwd: LoRA factors are NULL");
    XQ_REQUIRE(lora_dtype == XQ_DT_F32 || lora_dtype == XQ_DT_BF16, "xq_linear_bwd: bad lora_dtype");
    XQ_REQUIRE(!(dA || dB) || r > 0, "xq_linear_bwd: factor gradients requested with r == 0");
    XQ_REQUIRE(!(dA || dB) || M == 0 || x, "xq_linear_bwd: x is needed for the factor gradients");
    hipStream_t stream = (hipStream_t)stream_;
    const int rp = r_pad_of(r);
    if (M == 0) {
        if (dA && (rc = launch_zero_fill(dA, (int64_t)r * K * 4, stream))) return rc;
        if (dB && (rc = launch_zero_fill(dB, N * r * 4, stream))) return rc;
        return XQ_OK;
    }
    bf16_t *Bt = nullptr, *At = nullptr, *v = nullptr;
    const bf16_t* su = (const bf16_t*)su_in;
    float* partial = nullptr;
    Carver cv{(workspace && xq_aligned(workspace, 256)) ? (uint8_t*)workspace : nullptr, 0, workspace_bytes};
    if (rp) {
        XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= xq_linear_workspace_bytes(M, N, K, r),
                   "xq_linear_bwd: workspace missing, misaligned or smaller than xq_linear_workspace_bytes()");
        Bt = (bf16_t*)cv.take(rp * N * 2);
        At = (bf16_t*)cv.take(K * rp * 2);
        bf16_t* A_bf = (bf16_t*)cv.take(rp * K * 2);
        v = (bf16_t*)cv.take(M * rp * 2);
        bf16_t* su_ws = (bf16_t*)cv.take(M * rp * 2);
        // every factor layout this call needs, in one launch
        FactorPrepJobs jobs{};
        jobs.in_f32 = lora_dtype == XQ_DT_F32;
        jobs.add(lora_B, N, r, true, Bt, rp, N);
        if (dx) jobs.add(lora_A, r, K, true, At, K, rp);
        if (dB && !su) jobs.add(lora_A, r, K, false, A_bf, rp, K);
        if ((rc = launch_factor_prep_multi(jobs, stream))) return rc;
        // v = bf16(s * dy . B)   [M, rp]
        if ((rc = launch_small_nt((const bf16_t*)dy, lddy, M, N, Bt, rp, scaling, v, nullptr, nullptr, 1, true, stream))) return rc;
        if (dB && !su) {
            if ((rc = launch_small_nt((const bf16_t*)x, ldx, M, K, A_bf, rp, scaling, su_ws, nullptr, nullptr, 1, true, stream))) return rc;
            su = su_ws;
        }
    }
    // one region after the carved buffers: split-K partial sums of the dgrad first, then (stream order) the
    // partial sums of the factor gradients
    partial = (float*)cv.take(0);
    if (dx) {
        XQ_REQUIRE(lddx % 8 == 0 && xq_aligned(dx, 16), "xq_linear_bwd: dx rows must be 16-byte aligned");
        if ((rc = launch_tile_gemm(w, false, (const bf16_t*)dy, lddy, M, nullptr, nullptr, v, At, rp, nullptr, (bf16_t*)dx,
                                   lddx, stream, "xq_linear_bwd(dx)", partial, partial ? workspace_bytes - cv.used : 0)))
            return rc;
    }
    // dB[N, r] = dy^T . su ; dA[r, K] = (x^T . v)^T
    if (dB && (rc = launch_tn((const bf16_t*)dy, lddy, N, su, rp, r, M, false, dB, partial, nullptr, 1, stream))) return rc;
    if (dA && (rc = launch_tn((const bf16_t*)x, ldx, K, v, rp, r, M, true, dA, partial, nullptr, 1, stream))) return rc;
    return XQ_OK;
}

extern "C" int xq_grouped_gemm(const xq_weight* w, int transpose_w, const void* a, int64_t lda, int64_t n_rows,
                               const int32_t* offsets, const int32_t* tile_offsets, const void* su,
                               const void* lora_right, int r_pad, void* y, int64_t ldy, void* stream) {
    int rc = xq_validate_weight(w, "xq_grouped_gemm");
    if (rc) return rc;
    XQ_REQUIRE(offsets && tile_offsets, "xq_grouped_gemm: offsets / tile_offsets are NULL");
    XQ_REQUIRE(n_rows == 0 || (a && y), "xq_grouped_gemm: NULL activation pointer");
    XQ_REQUIRE(ldy % 8 == 0 && xq_aligned(y, 16), "xq_grouped_gemm: y rows must be 16-byte aligned");
    // bank is [E, K_in, N_out]: forward contracts over W rows, dgrad over W cols
    return launch_tile_gemm(w, transpose_w != 0, (const bf16_t*)a, lda, n_rows, offsets, tile_offsets, (const bf16_t*)su,
                            (const bf16_t*)lora_right, r_pad, nullptr, (bf16_t*)y, ldy, (hipStream_t)stream,
                            "xq_grouped_gemm", nullptr, 0);
}

extern "C" int xq_factor_prep(const void* in, int in_dtype, int64_t rows_in, int64_t cols_in, int transpose,
                              void* out_bf16, int64_t rows_out, int64_t cols_out, int64_t num_experts, void* stream) {
    XQ_REQUIRE(in_dtype == XQ_DT_F32 || in_dtype == XQ_DT_BF16, "xq_factor_prep: bad dtype");
    XQ_REQUIRE(num_experts == 0 || rows_out * cols_out == 0 || (in && out_bf16), "xq_factor_prep: NULL pointer");
    int64_t need_r = transpose ? cols_in : rows_in, need_c = transpose ? rows_in : cols_in;
    XQ_REQUIRE(rows_out >= need_r && cols_out >= need_c, "xq_factor_prep: output [%lld, %lld] smaller than source", (long long)rows_out, (long long)cols_out);
    return launch_factor_prep(in, in_dtype, rows_in, cols_in, transpose != 0, (bf16_t*)out_bf16, rows_out, cols_out,
                              num_experts, (hipStream_t)stream);
}

extern "C" int xq_grouped_lora_down(const void* a, int64_t lda, int64_t n_rows, const int32_t* offsets,
                                    const int32_t* tile_offsets, int32_t num_experts, const void* F, int shared,
                                    int r_pad, int64_t K, float scale, void* t, void* stream) {
    XQ_REQUIRE(offsets && tile_offsets && num_experts >= 1, "xq_grouped_lora_down: offsets / tile_offsets are NULL");
    XQ_REQUIRE(n_rows == 0 || (a && F && t), "xq_grouped_lora_down: NULL pointer");
    return launch_small_nt((const bf16_t*)a, lda, n_rows, K, (const bf16_t*)F, r_pad, scale, (bf16_t*)t, offsets,
                           tile_offsets, num_experts, shared != 0, (hipStream_t)stream);
}

extern "C" int64_t xq_lora_wgrad_workspace_bytes(int64_t n_rows, int64_t width, int r_pad) {
    return tn_partial_bytes(n_rows, width, r_pad) + 256;
}

extern "C" int xq_grouped_lora_wgrad(const void* P, int64_t ldp, int64_t p_width, const void* Q, int r_pad, int r_out,
                                     int64_t n_rows, const int32_t* offsets, int32_t num_experts, int transpose_out,
                                     float* out, void* workspace, const int32_t* row_limit, void* stream) {
    XQ_REQUIRE(out && (n_rows == 0 || (P && Q)), "xq_grouped_lora_wgrad: NULL pointer");
    if (n_rows == 0 && !offsets) return launch_zero_fill(out, p_width * r_out * 4, (hipStream_t)stream);
    return launch_tn((const bf16_t*)P, ldp, p_width, (const bf16_t*)Q, r_pad, r_out, n_rows, transpose_out != 0, out,
                     (float*)workspace, offsets, num_experts, (hipStream_t)stream, row_limit);
}
