// xq_grouped_fwd / xq_grouped_bwd: the routed SwiGLU expert MLP with LoRA on packed expert banks as two calls.
// Host code only: the program of the reference's _MoeExpertsLoRAFunction (ops/moe/lora.py:525-1007) composed from
// this library's kernels on the caller's stream -- routing, row movement, the fused dequant-GEMMs on the packed
// banks, the low-rank helpers and SwiGLU.  Nothing is allocated: temporaries are carved from the caller's workspace,
// tensors the backward needs live in caller buffers named by xq_grouped_saved.
#include "xq_lora.h"

namespace xq {
namespace {

inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }
inline int r_pad_of(int r) { return ((r + 15) / 16) * 16; }

struct Carve {
    uint8_t* base;
    int64_t used;
    template <typename T>
    T* take(int64_t bytes) {
        T* p = (T*)(base + used);
        used += al256(bytes);
        return p;
    }
};

// dst0[m][i][j] = src[m][i][j], dst1[m][i][j] = src[m][i][half + j] for j < r: the two factor gradients that one
// pass over the rows produced side by side
__global__ void __launch_bounds__(256) split_pair_kernel(const float* src, int64_t rows, int half, int r, float* dst0, float* dst1) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= rows * r) return;
    const int64_t i = t / r;
    const int j = (int)(t - i * r);
    dst0[t] = src[i * 2 * half + j];
    dst1[t] = src[i * 2 * half + half + j];
}

// token_of_row[scatter_index[i]] = i / topk: the token whose copy sits in row r of the expert order (routed copies
// with an invalid expert id have no row)
__global__ void __launch_bounds__(256) invert_scatter_kernel(const int32_t* scatter_index, int64_t n, int topk, int32_t* token_of_row) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int32_t r = scatter_index[i];
    if (r >= 0) token_of_row[r] = (int32_t)(i / topk);
}

struct Dims {
    int32_t E, topk, r, rp;
    int64_t T, R, H, I;
};

int check_call(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
               int64_t n_tokens, int32_t topk, const xq_grouped_saved* saved, const char* who, Dims* d) {
    XQ_REQUIRE(gate && up && down && lora && saved, "%s: NULL descriptor", who);
    int rc;
    if ((rc = xq_validate_weight(gate, who)) || (rc = xq_validate_weight(up, who)) || (rc = xq_validate_weight(down, who))) return rc;
    const int32_t E = gate->num_experts;
    XQ_REQUIRE(up->num_experts == E && down->num_experts == E, "%s: the three banks hold %d / %d / %d experts", who, E,
               up->num_experts, down->num_experts);
    const int64_t H = gate->rows, I = gate->cols;
    XQ_REQUIRE(up->rows == H && up->cols == I && down->rows == I && down->cols == H,
               "%s: bank shapes do not make an MLP (gate [%lld, %lld], up [%lld, %lld], down [%lld, %lld])", who,
               (long long)H, (long long)I, (long long)up->rows, (long long)up->cols, (long long)down->rows, (long long)down->cols);
    XQ_REQUIRE(H % 64 == 0 && I % 64 == 0, "%s: hidden size %lld and intermediate size %lld must be multiples of 64", who,
               (long long)H, (long long)I);
    XQ_REQUIRE(n_tokens >= 0 && topk >= 1 && n_tokens * topk < (1ll << 31), "%s: bad token count / top-k", who);
    XQ_REQUIRE(lora->r >= 1 && lora->r <= 64, "%s: LoRA rank %d out of range [1, 64]", who, lora->r);
    XQ_REQUIRE(lora->dtype == XQ_DT_F32 || lora->dtype == XQ_DT_BF16, "%s: bad lora dtype", who);
    for (int p = 0; p < 3; ++p) {
        XQ_REQUIRE(lora->A[p] && lora->B[p], "%s: LoRA factor %d is NULL", who, p);
        XQ_REQUIRE((lora->A_experts[p] == 1 || lora->A_experts[p] == E) && (lora->B_experts[p] == 1 || lora->B_experts[p] == E),
                   "%s: a LoRA factor holds 1 (shared) or %d matrices", who, E);
    }
    d->E = E; d->topk = topk; d->r = lora->r; d->rp = r_pad_of(lora->r);
    d->T = n_tokens; d->R = n_tokens * topk; d->H = H; d->I = I;
    if (d->R > 0)
        XQ_REQUIRE(saved->gate_up && saved->h && saved->w_row && saved->su_gate && saved->su_up &&
                       saved->su_down && saved->scatter_index,
                   "%s: a buffer of xq_grouped_saved is NULL", who);
    XQ_REQUIRE(saved->offsets && saved->tile_offsets && saved->counts, "%s: a routing buffer of xq_grouped_saved is NULL", who);
    return XQ_OK;
}

int64_t fwd_workspace(const Dims& d) {
    const int64_t panels = 2 * al256((int64_t)d.E * d.rp * d.H * 2) + 2 * al256((int64_t)d.E * d.I * d.rp * 2) +
                           al256((int64_t)d.E * d.rp * d.I * 2) + al256((int64_t)d.E * d.H * d.rp * 2);
    return al256(xq_route_workspace_bytes(d.R, d.E)) + panels + al256(d.R * d.H * 2) + al256(d.R * 4) + 256;
}

int64_t bwd_workspace(const Dims& d) {
    const int64_t EH = al256((int64_t)d.E * d.rp * d.H * 2), EI = al256((int64_t)d.E * d.rp * d.I * 2);
    const int64_t panels = 3 * EH + 3 * EI;     // F_dB, Lr_gA, Lr_uA over H; Lr_dA, F_gB, F_uB over I
    const int64_t wide = d.H > d.I ? d.H : d.I;
    const int64_t wg = al256(xq_lora_wgrad_workspace_bytes(d.R, wide, 2 * d.rp <= 64 ? 2 * d.rp : d.rp));
    const int64_t pair = al256((int64_t)d.E * d.H * 2 * d.rp * 4);      // the two A gradients side by side
    return panels + 3 * al256(d.R * d.H * 2) + al256(d.R * d.I * 2) + al256(d.R * 2 * d.I * 2) + 2 * al256(d.R * 4) +
           al256(d.R * d.rp * 2) + al256(d.R * 2 * d.rp * 2) + pair + wg + 256;
}

// one launch for gate and up (forward) / one sum for their two dgrads: block-fp8 banks on the pipelined kernel
bool fuse_gate_up(const xq_weight* gate, const xq_weight* up) { return two_banks_supported(gate) && two_banks_supported(up); }

}  // namespace
}  // namespace xq

using namespace xq;

extern "C" int xq_grouped_in_place(const xq_weight* gate, const xq_weight* up, const xq_weight* down) {
    (void)down;
    return gate && up && tile_gemm_takes_row_map(gate) && tile_gemm_takes_row_map(up) ? 1 : 0;
}

extern "C" int64_t xq_grouped_workspace_bytes(int64_t n_tokens, int32_t topk, int32_t num_experts, int64_t hidden,
                                              int64_t intermediate, int r, int backward) {
    if (n_tokens < 0 || topk < 1 || num_experts < 1 || r < 1) return 0;
    Dims d{num_experts, topk, r, r_pad_of(r), n_tokens, n_tokens * topk, hidden, intermediate};
    return backward ? bwd_workspace(d) : fwd_workspace(d);
}

extern "C" int xq_grouped_fwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                              const void* hidden, int64_t ld_hidden, int64_t n_tokens, const void* routing_w, int rw_dtype,
                              const int32_t* selected, int32_t topk, void* out, int64_t ld_out,
                              const xq_grouped_saved* saved, void* workspace, int64_t workspace_bytes, void* stream_) {
    static const char* who = "xq_grouped_fwd";
    Dims d;
    int rc = check_call(gate, up, down, lora, n_tokens, topk, saved, who, &d);
    if (rc) return rc;
    XQ_REQUIRE(rw_dtype == XQ_DT_F32 || rw_dtype == XQ_DT_BF16, "%s: routing weights are fp32 or bf16", who);
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= fwd_workspace(d),
               "%s: workspace missing, misaligned or smaller than xq_grouped_workspace_bytes()", who);
    XQ_REQUIRE(d.T == 0 || (hidden && routing_w && selected && out), "%s: NULL tensor", who);
    hipStream_t stream = (hipStream_t)stream_;
    const int E = d.E, rp = d.rp;
    const int64_t R = d.R, H = d.H, I = d.I;
    const float s = lora->scaling;
    const float limit = lora->swiglu_limit > 0.0f ? lora->swiglu_limit : 0.0f;
    Carve cv{(uint8_t*)workspace, 0};
    void* route_ws = cv.take<uint8_t>(xq_route_workspace_bytes(R, E));
    const int64_t route_ws_bytes = al256(xq_route_workspace_bytes(R, E));

    if ((rc = xq_route_build(selected, R, E, saved->counts, saved->offsets, saved->scatter_index, saved->tile_offsets,
                             route_ws, route_ws_bytes, stream)))
        return rc;
    if (R == 0) return XQ_OK;
    bf16_t* xs = (bf16_t*)saved->xs;
    // The pass that first reads the routed rows -- x . A^T of gate (and up) -- takes them from the token matrix through
    // the inverse of scatter_index and writes the expert-ordered copy xs on its way: no scatter pass of its own.
    // With saved->xs == NULL no copy is written at all: the projection launches read the token matrix through the same
    // map (the routed rows are rows of it, each topk times), and so does the backward (saved->x_tokens).
    int32_t* token_of_row = cv.take<int32_t>(R * 4);
    const bool ride = ld_hidden % 8 == 0 && xq_aligned(hidden, 16) && xq_aligned(xs, 16);
    const bool in_place = xs == nullptr;
    XQ_REQUIRE(!in_place || (ride && tile_gemm_takes_row_map(gate) && tile_gemm_takes_row_map(up)),
               "%s: saved->xs may be NULL only where xq_grouped_in_place() says so, with 16-byte aligned rows of hidden", who);
    if (ride) {
        invert_scatter_kernel<<<dim3((unsigned)xq_cdiv(R, 256)), 256, 0, stream>>>(saved->scatter_index, R, topk, token_of_row);
        XQ_CHECK_LAUNCH(who);
    } else if ((rc = xq_moe_scatter(hidden, ld_hidden, saved->scatter_index, R, topk, H, xs, H, stream))) {
        return rc;
    }
    const bf16_t* first_in = ride ? (const bf16_t*)hidden : xs;      // operand of the first pass
    const int64_t first_ld = ride ? ld_hidden : H;
    const int32_t* first_map = ride ? token_of_row : nullptr;
    bf16_t* first_copy = ride ? xs : nullptr;
    const bf16_t* xr = in_place ? (const bf16_t*)hidden : xs;         // the routed rows for the passes after the first
    const int64_t ld_xr = in_place ? ld_hidden : H;
    const int32_t* xr_rows = in_place ? token_of_row : nullptr;

    // bf16 operand layouts of the six factors, one launch.  A factors [E|1, in, r] become the "down" panels
    // [E|1, rp, in] of x . A; B factors [E|1, r, out] become the per-expert right-hand panels [E, out, rp].
    PanelJobs jobs{};
    jobs.in_f32 = lora->dtype == XQ_DT_F32;
    const int gAe = lora->A_experts[0], uAe = lora->A_experts[1], dAe = lora->A_experts[2];
    // gate's and up's A panels as the row bands [0, rp) and [rp, 2 rp) of one [2 rp, H] panel per expert when both are
    // held the same way: both low-rank intermediates then come from one pass over the routed rows
    const bool one_pass = gAe == uAe && 2 * rp <= 64;
    bf16_t *F_gA, *F_uA;
    if (one_pass) {
        F_gA = cv.take<bf16_t>((int64_t)gAe * 2 * rp * H * 2);
        F_uA = F_gA + (int64_t)rp * H;
        jobs.add(lora->A[0], gAe, H, d.r, true, F_gA, gAe, rp, H, 0, 2 * (int64_t)rp * H);
        jobs.add(lora->A[1], uAe, H, d.r, true, F_uA, uAe, rp, H, 0, 2 * (int64_t)rp * H);
    } else {
        F_gA = jobs.add(lora->A[0], gAe, H, d.r, true, cv.take<bf16_t>((int64_t)gAe * rp * H * 2), gAe, rp, H);
        F_uA = jobs.add(lora->A[1], uAe, H, d.r, true, cv.take<bf16_t>((int64_t)uAe * rp * H * 2), uAe, rp, H);
    }
    bf16_t* Lr_gB = jobs.add(lora->B[0], lora->B_experts[0], d.r, I, true, cv.take<bf16_t>((int64_t)E * I * rp * 2), E, I, rp);
    bf16_t* Lr_uB = jobs.add(lora->B[1], lora->B_experts[1], d.r, I, true, cv.take<bf16_t>((int64_t)E * I * rp * 2), E, I, rp);
    bf16_t* F_dA = jobs.add(lora->A[2], dAe, I, d.r, true, cv.take<bf16_t>((int64_t)dAe * rp * I * 2), dAe, rp, I);
    bf16_t* Lr_dB = jobs.add(lora->B[2], lora->B_experts[2], d.r, H, true, cv.take<bf16_t>((int64_t)E * H * rp * 2), E, H, rp);
    if ((rc = launch_panel_prep(jobs, stream))) return rc;
    bf16_t* down_out = cv.take<bf16_t>(R * H * 2);

    const int32_t *off = saved->offsets, *toff = saved->tile_offsets;
    bf16_t *su_g = (bf16_t*)saved->su_gate, *su_u = (bf16_t*)saved->su_up, *su_d = (bf16_t*)saved->su_down;
    bf16_t *gu = (bf16_t*)saved->gate_up, *h = (bf16_t*)saved->h;       // gu [R, 2I]: gate | up
    if (one_pass) {
        if ((rc = launch_small_nt(first_in, first_ld, R, H, F_gA, 2 * rp, s, su_g, off, toff, E, gAe == 1, stream, rp, su_u, rp,
                                  first_map, first_copy, H)))
            return rc;
    } else {
        if ((rc = launch_small_nt(first_in, first_ld, R, H, F_gA, rp, s, su_g, off, toff, E, gAe == 1, stream, 0, nullptr, 0,
                                  first_map, first_copy, H)))
            return rc;
        if ((rc = launch_small_nt(xr, ld_xr, R, H, F_uA, rp, s, su_u, off, toff, E, uAe == 1, stream, 0, nullptr, 0, xr_rows, nullptr, 0))) return rc;
    }
    if (fuse_gate_up(gate, up)) {       // both projections in one launch: column tiles past I take the up bank
        const TwoBanks two{up, su_u, Lr_uB};
        if ((rc = launch_tile_gemm(gate, false, xr, ld_xr, R, off, toff, su_g, Lr_gB, rp, nullptr, gu, 2 * I, stream, who, nullptr, 0, &two, xr_rows, d.T))) return rc;
    } else {
        if ((rc = launch_tile_gemm(gate, false, xr, ld_xr, R, off, toff, su_g, Lr_gB, rp, nullptr, gu, 2 * I, stream, who, nullptr, 0, nullptr, xr_rows, d.T))) return rc;
        if ((rc = launch_tile_gemm(up, false, xr, ld_xr, R, off, toff, su_u, Lr_uB, rp, nullptr, gu + I, 2 * I, stream, who, nullptr, 0, nullptr, xr_rows, d.T))) return rc;
    }
    if ((rc = xq_moe_scatter_scalar(routing_w, rw_dtype, saved->scatter_index, R, saved->w_row, stream))) return rc;
    // SwiGLU (times the row's routing weight) and s * h . A_d^T of the down projection: one pass where the rank allows
    static const bool silu_nt = [] { const char* e = getenv("XQ_MLP_SILU_NT"); return e ? atoi(e) != 0 : true; }();
    if (silu_nt && silu_bwd_nt_supported(I, rp)) {
        if ((rc = launch_silu_fwd_nt(gu, gu + I, 2 * I, h, I, R, I, F_dA, rp, s, su_d, rp, stream, off, toff, E, dAe == 1, saved->w_row, limit))) return rc;
    } else {
        if ((rc = silu_mul_fwd_limit(gu, gu + I, 2 * I, saved->w_row, h, I, R, I, limit, stream))) return rc;
        if ((rc = launch_small_nt(h, I, R, I, F_dA, rp, s, su_d, off, toff, E, dAe == 1, stream))) return rc;
    }
    if ((rc = launch_tile_gemm(down, false, h, I, R, off, toff, su_d, Lr_dB, rp, nullptr, down_out, H, stream, who, nullptr, 0))) return rc;
    return xq_moe_gather(down_out, nullptr, H, saved->scatter_index, d.T, topk, H, out, ld_out, stream);
}

extern "C" int xq_grouped_bwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                              const void* dy, int64_t ld_dy, int64_t n_tokens, int32_t topk, const xq_grouped_saved* saved,
                              void* dx, int64_t ld_dx, void* d_routing, int rw_dtype, const xq_grouped_grads* grads,
                              void* workspace, int64_t workspace_bytes, void* stream_) {
    static const char* who = "xq_grouped_bwd";
    Dims d;
    int rc = check_call(gate, up, down, lora, n_tokens, topk, saved, who, &d);
    if (rc) return rc;
    XQ_REQUIRE(grads, "%s: grads is NULL", who);
    for (int p = 0; p < 3; ++p) XQ_REQUIRE(grads->dA[p] && grads->dB[p], "%s: a factor gradient buffer is NULL", who);
    XQ_REQUIRE(!d_routing || rw_dtype == XQ_DT_F32 || rw_dtype == XQ_DT_BF16, "%s: routing-weight gradients are fp32 or bf16", who);
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= bwd_workspace(d),
               "%s: workspace missing, misaligned or smaller than xq_grouped_workspace_bytes()", who);
    hipStream_t stream = (hipStream_t)stream_;
    const int E = d.E, r = d.r, rp = d.rp;
    const int64_t R = d.R, H = d.H, I = d.I;
    const float s = lora->scaling;
    const float limit = lora->swiglu_limit > 0.0f ? lora->swiglu_limit : 0.0f;
    if (R == 0) {      // no rows: every factor gradient is zero
        for (int p = 0; p < 3; ++p) {
            const int64_t in = p == 2 ? I : H, outw = p == 2 ? H : I;
            if ((rc = launch_zero_fill(grads->dA[p], (int64_t)lora->A_experts[p] * in * r * 4, stream))) return rc;
            if ((rc = launch_zero_fill(grads->dB[p], (int64_t)lora->B_experts[p] * r * outw * 4, stream))) return rc;
        }
        return XQ_OK;
    }
    XQ_REQUIRE(dy, "%s: dy is NULL", who);
    Carve cv{(uint8_t*)workspace, 0};
    const int32_t *off = saved->offsets, *toff = saved->tile_offsets, *sidx = saved->scatter_index;
    const int32_t* n_valid = off + E;     // rows that belong to an expert (all of them unless an id was out of range)
    const bf16_t *xs = (const bf16_t*)saved->xs, *gu = (const bf16_t*)saved->gate_up;
    // the forward kept no expert-ordered copy of the routed rows: they are read from the token matrix through the map
    const bool x_in_place = xs == nullptr;
    XQ_REQUIRE(!x_in_place || (saved->x_tokens && saved->ld_x_tokens % 8 == 0 && xq_aligned(saved->x_tokens, 16)),
               "%s: saved->xs is NULL and saved->x_tokens does not name the forward's hidden states (16-byte aligned rows)", who);
    const bf16_t *h = (const bf16_t*)saved->h, *su_g = (const bf16_t*)saved->su_gate, *su_u = (const bf16_t*)saved->su_up;
    const bf16_t* su_d = (const bf16_t*)saved->su_down;
    const int gBe = lora->B_experts[0], uBe = lora->B_experts[1], dBe = lora->B_experts[2];
    const int gAe = lora->A_experts[0], uAe = lora->A_experts[1], dAe = lora->A_experts[2];
    // one dgrad launch for gate and up: dX = [dgate | dup] . [Wg ; Wu]^T + [v_g | v_u] . [Lr_gA | Lr_uA]^T (the two
    // low-rank terms ride as one side term of width 2 * rp)
    // (the A gradients then come from one pass over the rows too, which wants both A factors held the same way)
    const bool fused = fuse_gate_up(gate, up) && 2 * rp <= 64 && gAe == uAe;
    const int rp2 = 2 * rp;

    // every panel of the call in one launch: B factors [E|1, r, out] as the "down" panels [E|1, rp, out] of g . B^T,
    // A factors [E|1, in, r] as the per-expert right-hand panels [E, in, rp] of the dgrads (gate's and up's side by
    // side in one [E, H, 2 rp] panel when their dgrads share a launch)
    PanelJobs jobs{};
    jobs.in_f32 = lora->dtype == XQ_DT_F32;
    bf16_t* F_dB = jobs.add(lora->B[2], dBe, r, H, false, cv.take<bf16_t>((int64_t)dBe * rp * H * 2), dBe, rp, H);
    bf16_t* Lr_dA = jobs.add(lora->A[2], dAe, I, r, false, cv.take<bf16_t>((int64_t)E * I * rp * 2), E, I, rp);
    bf16_t* F_uB = jobs.add(lora->B[1], uBe, r, I, false, cv.take<bf16_t>((int64_t)uBe * rp * I * 2), uBe, rp, I);
    bf16_t* F_gB = jobs.add(lora->B[0], gBe, r, I, false, cv.take<bf16_t>((int64_t)gBe * rp * I * 2), gBe, rp, I);
    bf16_t* Lr_guA = cv.take<bf16_t>((int64_t)E * H * rp2 * 2);       // fused: [E, H, 2 rp]; else gate's [E, H, rp] then up's
    bf16_t* Lr_uA = fused ? Lr_guA + rp : Lr_guA + (int64_t)E * H * rp;
    jobs.add(lora->A[0], gAe, H, r, false, Lr_guA, E, H, rp, fused ? rp2 : rp);
    jobs.add(lora->A[1], uAe, H, r, false, Lr_uA, E, H, rp, fused ? rp2 : rp);
    if ((rc = launch_panel_prep(jobs, stream))) return rc;

    bf16_t* g_down = cv.take<bf16_t>(R * H * 2);
    bf16_t* dx_g = cv.take<bf16_t>(R * H * 2);
    bf16_t* dx_u = cv.take<bf16_t>(R * H * 2);
    bf16_t* dh = cv.take<bf16_t>(R * I * 2);
    bf16_t* dgu = cv.take<bf16_t>(R * 2 * I * 2);         // [R, 2I]: dgate | dup
    float* d_w_row = cv.take<float>(R * 4);
    bf16_t* v_d = cv.take<bf16_t>(R * rp * 2);
    bf16_t* v_gu = cv.take<bf16_t>(R * rp2 * 2);          // fused: [R, 2 rp] = v_g | v_u; else v_g [R, rp] then v_u [R, rp]
    float* pair = cv.take<float>((int64_t)E * H * rp2 * 4);
    int32_t* token_of_row = cv.take<int32_t>(R * 4);
    float* wg = cv.take<float>(0);
    bf16_t *dgate = dgu, *dup = dgu + I;
    bf16_t* v_g = v_gu;
    bf16_t* v_u = fused ? v_gu + rp : v_gu + R * rp;
    const int64_t ld_v = fused ? rp2 : rp;

    // The routed gradient rows are rows of dy, each of them topk times: with 16-byte aligned rows nothing expert-ordered is
    // written for them -- the passes that read them (s * g . B^T, the dgrad launch, the B gradient) go through the inverse of
    // scatter_index to dy itself, 1 / topk of the bytes and mostly cache hits.  (A bank that takes the generic tile kernel
    // still gets its copy, written by the first pass on its way.)
    const bool ride = ld_dy % 8 == 0 && xq_aligned(dy, 16);
    const bool in_place = ride && tile_gemm_takes_row_map(down);
    if (x_in_place && !ride) {
        invert_scatter_kernel<<<dim3((unsigned)xq_cdiv(R, 256)), 256, 0, stream>>>(sidx, R, topk, token_of_row);
        XQ_CHECK_LAUNCH(who);
    }
    const bf16_t* xr = x_in_place ? (const bf16_t*)saved->x_tokens : xs;
    const int64_t ld_xr = x_in_place ? saved->ld_x_tokens : H;
    const int32_t* xr_rows = x_in_place ? token_of_row : nullptr;
    if (ride) {
        invert_scatter_kernel<<<dim3((unsigned)xq_cdiv(R, 256)), 256, 0, stream>>>(sidx, R, topk, token_of_row);
        XQ_CHECK_LAUNCH(who);
    } else if ((rc = xq_moe_scatter(dy, ld_dy, sidx, R, topk, H, g_down, H, stream))) {
        return rc;
    }

    // ---- down projection: y = h.W + s*(h.A).B
    if ((rc = launch_small_nt(ride ? (const bf16_t*)dy : g_down, ride ? ld_dy : H, R, H, F_dB, rp, s, v_d, off, toff, E, dBe == 1, stream,
                              0, nullptr, 0, ride ? token_of_row : nullptr, ride && !in_place ? g_down : nullptr, H)))        // s * g . B^T
        return rc;
    const bf16_t* gd = in_place ? (const bf16_t*)dy : g_down;      // the routed gradient rows: dy through the map, or the copy
    const int64_t ld_gd = in_place ? ld_dy : H;
    const int32_t* gd_rows = in_place ? token_of_row : nullptr;
    if ((rc = launch_tile_gemm(down, true, gd, ld_gd, R, off, toff, v_d, Lr_dA, rp, nullptr, dh, I, stream, who, nullptr, 0, nullptr, gd_rows, d.T))) return rc;
    if ((rc = launch_tn(gd, ld_gd, H, su_d, rp, r, R, true, grads->dB[2], wg, dBe == 1 ? nullptr : off, E, stream, n_valid, 0, gd_rows))) return rc;   // [E|1, r, H]
    if ((rc = launch_tn(h, I, I, v_d, rp, r, R, false, grads->dA[2], wg, dAe == 1 ? nullptr : off, E, stream, n_valid))) return rc;        // [E|1, I, r]

    // ---- SwiGLU + routing weight, and s * dgate . B_g^T, s * dup . B_u^T of the up / gate projections (y = x.W + s*(x.A).B):
    // one pass over (gate, up, dh) where the rank allows, so that the two products do not read dgate | dup back
    static const bool silu_nt = [] { const char* e = getenv("XQ_MLP_SILU_NT"); return e ? atoi(e) != 0 : true; }();
    if (silu_nt && silu_bwd_nt_supported(I, rp)) {
        if ((rc = launch_silu_bwd_nt(gu, gu + I, 2 * I, dh, I, dgate, dup, 2 * I, R, I, F_gB, F_uB, rp, s, v_g, v_u, ld_v, stream, off, toff, E,
                                     gBe == 1, uBe == 1, saved->w_row, d_w_row, limit)))
            return rc;
    } else {
        if ((rc = silu_mul_bwd_limit(gu, gu + I, 2 * I, dh, I, saved->w_row, dgate, dup, 2 * I, d_w_row, R, I, limit, stream))) return rc;
        if ((rc = launch_small_nt(dup, 2 * I, R, I, F_uB, rp, s, v_u, off, toff, E, uBe == 1, stream, ld_v))) return rc;
        if ((rc = launch_small_nt(dgate, 2 * I, R, I, F_gB, rp, s, v_g, off, toff, E, gBe == 1, stream, ld_v))) return rc;
    }
    if (d_routing && (rc = xq_moe_gather_scalar(d_w_row, sidx, R, d_routing, rw_dtype, stream))) return rc;
    if (fused) {
        const TwoBanks two{up, nullptr, nullptr};
        if ((rc = launch_tile_gemm(gate, true, dgu, 2 * I, R, off, toff, v_gu, Lr_guA, rp2, nullptr, dx_g, H, stream, who, nullptr, 0, &two))) return rc;
    } else {
        if ((rc = launch_tile_gemm(up, true, dup, 2 * I, R, off, toff, v_u, Lr_uA, rp, nullptr, dx_u, H, stream, who, nullptr, 0))) return rc;
        if ((rc = launch_tile_gemm(gate, true, dgate, 2 * I, R, off, toff, v_g, Lr_guA, rp, nullptr, dx_g, H, stream, who, nullptr, 0))) return rc;
    }
    if ((rc = launch_tn(dup, 2 * I, I, su_u, rp, r, R, true, grads->dB[1], wg, uBe == 1 ? nullptr : off, E, stream, n_valid))) return rc;      // [E|1, r, I]
    if ((rc = launch_tn(dgate, 2 * I, I, su_g, rp, r, R, true, grads->dB[0], wg, gBe == 1 ? nullptr : off, E, stream, n_valid))) return rc;
    // gradients of the two A factors, [E|1, H, r] = x^T . v: both contract the same rows of x, so with v_g | v_u side
    // by side they share one pass over them
    if (fused) {
        if ((rc = launch_tn(xr, ld_xr, H, v_gu, rp2, rp2, R, false, pair, wg, gAe == 1 ? nullptr : off, E, stream, n_valid, 0, xr_rows))) return rc;
        const int64_t rows = (int64_t)gAe * H;
        split_pair_kernel<<<dim3((unsigned)xq_cdiv(rows * r, 256)), 256, 0, stream>>>(pair, rows, rp, r, grads->dA[0], grads->dA[1]);
        XQ_CHECK_LAUNCH(who);
    } else {
        if ((rc = launch_tn(xr, ld_xr, H, v_g, rp, r, R, false, grads->dA[0], wg, gAe == 1 ? nullptr : off, E, stream, n_valid, 0, xr_rows))) return rc;
        if ((rc = launch_tn(xr, ld_xr, H, v_u, rp, r, R, false, grads->dA[1], wg, uAe == 1 ? nullptr : off, E, stream, n_valid, 0, xr_rows))) return rc;
    }
    if (!dx) return XQ_OK;
    return xq_moe_gather(dx_g, fused ? nullptr : dx_u, H, sidx, d.T, topk, H, dx, ld_dx, stream);
}
