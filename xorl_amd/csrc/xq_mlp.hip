// xq_mlp_fwd / xq_mlp_bwd: the dense SwiGLU MLP of three QLoRA linears (gate, up, down) as two calls.
// Host code only.  The program is the reference's Qwen3MLP.forward over three QLoRALinear modules
// (models/transformers/qwen3/modeling_qwen3.py:60-81 with qlora/modules/linear.py:369-385 and
// ops/fused_silu_and_mul.py:22-60) and its backward, composed from this library's kernels on the caller's stream
// so that work the three separate module calls repeat is shared:
//   forward   one pass over x gives both low-rank intermediates; block-fp8 gate / up run as one launch whose
//             epilogue also writes h = bf16(silu(gate)) * up;
//   backward  the dgrads of gate and up are one launch, dX = [dgate | dup] . [Wg ; Wu] + [v_g | v_u] . [A_g ; A_u],
//             and the two A gradients come from one pass over x.
// Other formats (and shapes the fused forms do not take) run the same program launch by launch.
#include "xq_lora.h"
#include <atomic>
#include <stdlib.h>

namespace xq {
namespace {

inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }
inline int r_pad_of(int r) { return r <= 0 ? 0 : ((r + 15) / 16) * 16; }

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

struct Dims {
    int64_t M, H, I;
    int r, rp;
};

// dst[j][c] = src[j0 + j][c] for j < rows: the two factor gradients that one pass over x left in one matrix
__global__ void __launch_bounds__(256) copy_rows_kernel(const float* src, int64_t width, int j0, int rows, float* dst) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t < (int64_t)rows * width) dst[t] = src[(int64_t)j0 * width + t];
}

// a[m][c] = bf16(a[m][c] + b[m][c]): the two shares of dX when the dgrads of gate and up run as separate launches
__global__ void __launch_bounds__(256) add_rows_kernel(bf16_t* a, int64_t lda, const bf16_t* b, int64_t ldb, int64_t rows, int64_t cols8) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= rows * cols8) return;
    const int64_t m = t / cols8, c = (t - m * cols8) * 8;
    u32x4 av = *(const u32x4*)(a + m * lda + c), bv = *(const u32x4*)(b + m * ldb + c), o;
#pragma unroll
    for (int i = 0; i < 4; ++i)
        o[i] = pack_bf16x2(bf16_to_f32((bf16_t)(av[i] & 0xffffu)) + bf16_to_f32((bf16_t)(bv[i] & 0xffffu)),
                           bf16_to_f32((bf16_t)(av[i] >> 16)) + bf16_to_f32((bf16_t)(bv[i] >> 16)));
    *(u32x4*)(a + m * lda + c) = o;
}

// gate and up of a block-fp8 MLP as ONE launch with the SwiGLU in its epilogue (1), or as two launches followed by the pass
// that writes h and forms s * h . A_d^T on the way (0, the default: the two plain launches run at a higher rate than the
// launch with the wide epilogue, and the step is level or slightly shorter).  XQ_MLP_GU in the environment sets it at load
// time, xq_set_mlp_gate_up_fused() at run time.  It is only the default of a forward: xq_mlp_saved::gate_up_fused carries the
// form a forward used (or was asked for) to its backward, which lays out the saved low-rank intermediates by that field.
static std::atomic<int> g_mlp_gu{[] { const char* e = getenv("XQ_MLP_GU"); return e ? atoi(e) : 0; }()};
// XQ_MLP_SILU_NT=0: the SwiGLU backward and the two low-rank products of its outputs as three launches (A/B measurements;
// same bits either way)
static const int g_mlp_silu_nt = [] { const char* e = getenv("XQ_MLP_SILU_NT"); return e ? atoi(e) : 1; }();
// `asked`: xq_mlp_saved::gate_up_fused on entry to the forward (< 0: the process-wide default decides)
bool fuse_gate_up_fwd(const xq_weight* gate, const xq_weight* up, int asked) {
    return (asked < 0 ? g_mlp_gu.load() != 0 : asked != 0) && gate->format == XQ_FMT_FP8 && up->format == XQ_FMT_FP8;
}

// Where the two low-rank intermediates lie in su_gate_up (M * 2 * rp elements): as the column bands [0, rp) and
// [rp, 2 rp) of one [M, 2 rp] matrix when the fused gate / up launch reads them, else as two packed [M, rp] matrices.
struct SuLayout {
    int64_t up_offset, pitch;
};
SuLayout su_layout(bool fused_fwd, int rp, int64_t M) {
    if (fused_fwd) return {rp, 2 * (int64_t)rp};
    return {M * rp, rp};
}

int check_call(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora, int64_t M,
               const xq_mlp_saved* saved, const char* who, Dims* d) {
    XQ_REQUIRE(gate && up && down && lora && saved, "%s: NULL descriptor", who);
    int rc;
    if ((rc = xq_validate_weight(gate, who)) || (rc = xq_validate_weight(up, who)) || (rc = xq_validate_weight(down, who))) return rc;
    for (const xq_weight* w : {gate, up, down}) {
        XQ_REQUIRE(w->num_experts == 1, "%s: dense weights only", who);
        XQ_REQUIRE(w->format == XQ_FMT_FP8 || w->layout == XQ_LAYOUT_FLAT, "%s: dense weights are FLAT [out, in]", who);
    }
    const int64_t I = gate->rows, H = gate->cols;
    XQ_REQUIRE(up->rows == I && up->cols == H && down->rows == H && down->cols == I,
               "%s: weight shapes do not make an MLP (gate [%lld, %lld], up [%lld, %lld], down [%lld, %lld])", who, (long long)I,
               (long long)H, (long long)up->rows, (long long)up->cols, (long long)down->rows, (long long)down->cols);
    XQ_REQUIRE(H % 64 == 0 && I % 64 == 0, "%s: hidden size %lld and intermediate size %lld must be multiples of 64", who,
               (long long)H, (long long)I);
    XQ_REQUIRE(M >= 0, "%s: negative row count", who);
    XQ_REQUIRE(lora->r >= 0 && lora->r <= 64, "%s: LoRA rank %d out of range [0, 64]", who, lora->r);
    XQ_REQUIRE(lora->dtype == XQ_DT_F32 || lora->dtype == XQ_DT_BF16, "%s: bad lora dtype", who);
    if (lora->r > 0)
        for (int p = 0; p < 3; ++p) XQ_REQUIRE(lora->A[p] && lora->B[p], "%s: LoRA factor %d is NULL", who, p);
    d->M = M; d->H = H; d->I = I; d->r = lora->r; d->rp = r_pad_of(lora->r);
    if (M > 0) XQ_REQUIRE(saved->gate_up && saved->h && (d->rp == 0 || (saved->su_gate_up && saved->su_down)), "%s: a buffer of xq_mlp_saved is NULL", who);
    XQ_REQUIRE(xq_aligned(saved->gate_up, 16) && xq_aligned(saved->h, 16), "%s: gate_up and h of xq_mlp_saved must be 16-byte aligned", who);
    for (int p = 0; p < 3; ++p) XQ_REQUIRE(xq_aligned(lora->bias[p], 8), "%s: bias vectors must be 8-byte aligned", who);
    return XQ_OK;
}

int64_t fwd_workspace(const Dims& d) {
    const int64_t rp = d.rp ? d.rp : 16;
    const int64_t pa = tile_gemm_partial_bytes(d.M, d.I, d.H), pb = tile_gemm_partial_bytes(d.M, d.H, d.I);
    return al256(2 * rp * d.H * 2) + 2 * al256(d.I * rp * 2) + al256(rp * d.I * 2) + al256(d.H * rp * 2) + al256(pa > pb ? pa : pb) + 512;
}

int64_t bwd_workspace(const Dims& d) {
    const int64_t rp = d.rp ? d.rp : 16, wide = d.H > d.I ? d.H : d.I;
    const int64_t panels = al256(rp * d.H * 2) + al256(d.I * rp * 2) + 2 * al256(rp * d.I * 2) + al256(d.H * 2 * rp * 2);
    int64_t tn = tn_partial_bytes(d.M, wide, 2 * rp <= 64 ? 2 * rp : rp);
    const int64_t pa = tile_gemm_partial_bytes(d.M, d.I, d.H), pb = tile_gemm_partial_bytes(d.M, d.H, d.I);
    tn = tn > pa ? tn : pa;
    tn = tn > pb ? tn : pb;
    return panels + al256(d.M * d.I * 2) + al256(d.M * 2 * d.I * 2) + al256(d.M * d.H * 2) + al256(d.M * rp * 2) +
           al256(d.M * 2 * rp * 2) + al256(2 * rp * d.H * 4) + al256(tn) + 512;
}

}  // namespace
}  // namespace xq

using namespace xq;

extern "C" int xq_set_mlp_gate_up_fused(int enabled) {
    g_mlp_gu = enabled != 0;
    return XQ_OK;
}

extern "C" int xq_get_mlp_gate_up_fused(void) { return g_mlp_gu.load() != 0; }

extern "C" int64_t xq_mlp_workspace_bytes(int64_t M, int64_t hidden, int64_t intermediate, int r, int backward) {
    if (M < 0 || r < 0) return 0;
    Dims d{M, hidden, intermediate, r, r_pad_of(r)};
    return backward ? bwd_workspace(d) : fwd_workspace(d);
}

extern "C" int xq_mlp_fwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
                          const void* x_, int64_t ldx, int64_t M, void* y, int64_t ldy, xq_mlp_saved* saved,
                          void* workspace, int64_t workspace_bytes, void* stream_) {
    static const char* who = "xq_mlp_fwd";
    Dims d;
    int rc = check_call(gate, up, down, lora, M, saved, who, &d);
    if (rc) return rc;
    const bool fused = fuse_gate_up_fwd(gate, up, saved->gate_up_fused);
    saved->gate_up_fused = fused ? 1 : 0;       // what the backward must be told
    if (M == 0) return XQ_OK;
    XQ_REQUIRE(x_ && y, "%s: NULL activation pointer", who);
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= fwd_workspace(d),
               "%s: workspace missing, misaligned or smaller than xq_mlp_workspace_bytes()", who);
    XQ_REQUIRE(ldy % 8 == 0 && xq_aligned(y, 16), "%s: y rows must be 16-byte aligned", who);
    hipStream_t stream = (hipStream_t)stream_;
    const bf16_t* x = (const bf16_t*)x_;
    const int r = d.r, rp = d.rp;
    const int64_t H = d.H, I = d.I;
    const float s = lora->scaling;
    bf16_t *gu = (bf16_t*)saved->gate_up, *h = (bf16_t*)saved->h;
    bf16_t *su_gu = (bf16_t*)saved->su_gate_up, *su_d = (bf16_t*)saved->su_down;
    Carve cv{(uint8_t*)workspace, 0};
    bf16_t *A_gu = nullptr, *Bl_g = nullptr, *Bl_u = nullptr, *A_d = nullptr, *Bl_d = nullptr;
    const SuLayout sl = su_layout(fused, rp, M);
    const bool one_pass = fused && rp > 0 && 2 * rp <= 64;      // both low-rank intermediates from one pass over x
    if (rp) {
        // panels: [A_g ; A_u] as [2 rp, H] (the rows of x . A^T), B as [out, rp] right-hand panels
        PanelJobs jobs{};
        jobs.in_f32 = lora->dtype == XQ_DT_F32;
        A_gu = cv.take<bf16_t>(2 * rp * H * 2);
        jobs.add(lora->A[0], 1, r, H, false, A_gu, 1, rp, H);
        jobs.add(lora->A[1], 1, r, H, false, A_gu + (int64_t)rp * H, 1, rp, H);
        Bl_g = jobs.add(lora->B[0], 1, I, r, false, cv.take<bf16_t>(I * rp * 2), 1, I, rp);
        Bl_u = jobs.add(lora->B[1], 1, I, r, false, cv.take<bf16_t>(I * rp * 2), 1, I, rp);
        A_d = jobs.add(lora->A[2], 1, r, I, false, cv.take<bf16_t>(rp * I * 2), 1, rp, I);
        Bl_d = jobs.add(lora->B[2], 1, H, r, false, cv.take<bf16_t>(H * rp * 2), 1, H, rp);
        if ((rc = launch_panel_prep(jobs, stream))) return rc;
        // bf16(s * x . A^T) of gate and up
        if (one_pass) {
            if ((rc = launch_small_nt(x, ldx, M, H, A_gu, 2 * rp, s, su_gu, nullptr, nullptr, 1, true, stream))) return rc;
        } else {
            if ((rc = launch_small_nt(x, ldx, M, H, A_gu, rp, s, su_gu, nullptr, nullptr, 1, true, stream, sl.pitch))) return rc;
            if ((rc = launch_small_nt(x, ldx, M, H, A_gu + (int64_t)rp * H, rp, s, su_gu + sl.up_offset, nullptr, nullptr, 1, true, stream, sl.pitch))) return rc;
        }
    }
    float* part = cv.take<float>(0);
    const int64_t part_bytes = workspace_bytes - cv.used;
    const bf16_t *bias_g = (const bf16_t*)lora->bias[0], *bias_u = (const bf16_t*)lora->bias[1], *bias_d = (const bf16_t*)lora->bias[2];
    bool h_product_done = false;
    if (fused) {
        if ((rc = launch_gate_up_swiglu(gate, up, x, ldx, M, rp ? su_gu : nullptr, rp ? su_gu + sl.up_offset : nullptr, sl.pitch, Bl_g, Bl_u,
                                        rp, bias_g, bias_u, gu, 2 * I, h, I, stream)))
            return rc;
    } else {
        if ((rc = launch_tile_gemm(gate, true, x, ldx, M, nullptr, nullptr, rp ? su_gu : nullptr, Bl_g, rp, bias_g, gu, 2 * I, stream, who, part, part_bytes))) return rc;
        if ((rc = launch_tile_gemm(up, true, x, ldx, M, nullptr, nullptr, rp ? su_gu + sl.up_offset : nullptr, Bl_u, rp, bias_u, gu + I, 2 * I, stream, who, part, part_bytes))) return rc;
        // SwiGLU, and s * h . A_d^T of the down projection from the values on their way out where the rank allows
        if (rp && g_mlp_silu_nt && silu_bwd_nt_supported(I, rp)) {
            if ((rc = launch_silu_fwd_nt(gu, gu + I, 2 * I, h, I, M, I, A_d, rp, s, su_d, rp, stream))) return rc;
            h_product_done = true;
        } else if ((rc = xq_silu_mul_fwd(gu, gu + I, 2 * I, nullptr, h, I, M, I, stream))) {
            return rc;
        }
    }
    if (rp && !h_product_done && (rc = launch_small_nt(h, I, M, I, A_d, rp, s, su_d, nullptr, nullptr, 1, true, stream))) return rc;
    return launch_tile_gemm(down, true, h, I, M, nullptr, nullptr, rp ? su_d : nullptr, Bl_d, rp, bias_d, (bf16_t*)y, ldy, stream,
                            who, part, part_bytes);
}

// ---- forward only: nothing is kept for a backward, so each projection is free to take the kernel that suits the row
// count -- at decode sizes the weight-streaming kernels (gate and up as one launch), not the tile kernels above
static int64_t infer_linear_ws(int64_t M, int64_t H, int64_t I, int r) {
    const int64_t a = xq_linear_workspace_bytes(M, I, H, r), b = xq_linear_workspace_bytes(M, H, I, r);
    return al256((a > b ? a : b) > 2048 ? (a > b ? a : b) : 2048);
}

extern "C" int64_t xq_mlp_infer_workspace_bytes(int64_t M, int64_t hidden, int64_t intermediate, int r) {
    if (M < 0 || r < 0) return 0;
    return al256(M * 2 * intermediate * 2) + al256(M * intermediate * 2) + infer_linear_ws(M, hidden, intermediate, r) + 256;
}

extern "C" int xq_mlp_fwd_infer(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
                                const void* x, int64_t ldx, int64_t M, void* y, int64_t ldy, void* workspace,
                                int64_t workspace_bytes, void* stream) {
    static const char* who = "xq_mlp_fwd_infer";
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256), "%s: workspace missing or misaligned", who);
    Dims d;
    Carve cv{(uint8_t*)workspace, 0};
    // (the argument checks are those of xq_mlp_fwd; the buffers it would keep for a backward live in the workspace here)
    xq_mlp_saved tmp{workspace, workspace, workspace, workspace, 0, 0};
    int rc = check_call(gate, up, down, lora, M, &tmp, who, &d);
    if (rc) return rc;
    if (M == 0) return XQ_OK;
    XQ_REQUIRE(x && y, "%s: NULL activation pointer", who);
    XQ_REQUIRE(workspace_bytes >= xq_mlp_infer_workspace_bytes(M, d.H, d.I, d.r),
               "%s: workspace smaller than xq_mlp_infer_workspace_bytes()", who);
    bf16_t* gu = cv.take<bf16_t>(M * 2 * d.I * 2);
    bf16_t* h = cv.take<bf16_t>(M * d.I * 2);
    void* ws = cv.take<uint8_t>(0);
    const int64_t ws_bytes = workspace_bytes - cv.used;
    xq_linear_job jobs[2] = {
        {gate, lora->A[0], lora->B[0], d.r, lora->scaling, lora->bias[0], gu, 2 * d.I},
        {up, lora->A[1], lora->B[1], d.r, lora->scaling, lora->bias[1], gu + d.I, 2 * d.I},
    };
    if ((rc = xq_linear_fwd_multi(jobs, 2, x, ldx, M, lora->dtype, ws, ws_bytes, stream))) return rc;
    if ((rc = xq_silu_mul_fwd(gu, gu + d.I, 2 * d.I, nullptr, h, d.I, M, d.I, stream))) return rc;
    return xq_linear_fwd(down, h, d.I, M, lora->A[2], lora->B[2], lora->dtype, d.r, lora->scaling, lora->bias[2], y, ldy, nullptr, ws,
                         ws_bytes, stream);
}

extern "C" int xq_mlp_bwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
                          const void* x_, int64_t ldx, const void* dy_, int64_t lddy, int64_t M, const xq_mlp_saved* saved,
                          void* dx, int64_t lddx, const xq_mlp_grads* grads, void* workspace, int64_t workspace_bytes,
                          void* stream_) {
    static const char* who = "xq_mlp_bwd";
    Dims d;
    int rc = check_call(gate, up, down, lora, M, saved, who, &d);
    if (rc) return rc;
    const int r = d.r, rp = d.rp;
    const int64_t H = d.H, I = d.I;
    XQ_REQUIRE(saved->gate_up_fused == 0 || (saved->gate_up_fused == 1 && gate->format == XQ_FMT_FP8 && up->format == XQ_FMT_FP8),
               "%s: xq_mlp_saved::gate_up_fused is %d: pass the struct the forward filled (0 or 1; 1 only for block-fp8 gate and up)", who,
               saved->gate_up_fused);
    XQ_REQUIRE(rp == 0 || grads, "%s: grads is NULL", who);
    if (rp) for (int p = 0; p < 3; ++p) XQ_REQUIRE(grads->dA[p] && grads->dB[p], "%s: a factor gradient buffer is NULL", who);
    hipStream_t stream = (hipStream_t)stream_;
    if (M == 0) {
        for (int p = 0; p < 3 && rp; ++p) {
            const int64_t in = p == 2 ? I : H, outw = p == 2 ? H : I;
            if ((rc = launch_zero_fill(grads->dA[p], (int64_t)r * in * 4, stream))) return rc;
            if ((rc = launch_zero_fill(grads->dB[p], outw * r * 4, stream))) return rc;
        }
        return XQ_OK;
    }
    XQ_REQUIRE(x_ && dy_, "%s: NULL activation pointer", who);
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= bwd_workspace(d),
               "%s: workspace missing, misaligned or smaller than xq_mlp_workspace_bytes()", who);
    XQ_REQUIRE(!dx || (lddx % 8 == 0 && xq_aligned(dx, 16)), "%s: dx rows must be 16-byte aligned", who);
    const bf16_t *x = (const bf16_t*)x_, *dy = (const bf16_t*)dy_;
    const float s = lora->scaling;
    const bf16_t *gu = (const bf16_t*)saved->gate_up, *h = (const bf16_t*)saved->h;
    const bf16_t *su_gu = (const bf16_t*)saved->su_gate_up, *su_d = (const bf16_t*)saved->su_down;
    const int rp2 = 2 * rp;
    // one dgrad launch for gate and up (block-fp8, side term of width 2 rp)
    const bool fused = two_dense_supported(gate) && two_dense_supported(up) && rp2 <= 64;

    Carve cv{(uint8_t*)workspace, 0};
    bf16_t *Bt_d = nullptr, *At_d = nullptr, *Bt_g = nullptr, *Bt_u = nullptr, *At_gu = nullptr;
    if (rp) {
        PanelJobs jobs{};
        jobs.in_f32 = lora->dtype == XQ_DT_F32;
        Bt_d = jobs.add(lora->B[2], 1, H, r, true, cv.take<bf16_t>(rp * H * 2), 1, rp, H);          // [rp, H]: rows of dy . B
        At_d = jobs.add(lora->A[2], 1, r, I, true, cv.take<bf16_t>(I * rp * 2), 1, I, rp);          // [I, rp]: right-hand panel of the dgrad
        Bt_g = jobs.add(lora->B[0], 1, I, r, true, cv.take<bf16_t>(rp * I * 2), 1, rp, I);
        Bt_u = jobs.add(lora->B[1], 1, I, r, true, cv.take<bf16_t>(rp * I * 2), 1, rp, I);
        At_gu = cv.take<bf16_t>(H * rp2 * 2);            // fused: [H, 2 rp] = A_g^T | A_u^T; else A_g^T [H, rp] then A_u^T [H, rp]
        jobs.add(lora->A[0], 1, r, H, true, At_gu, 1, H, rp, fused ? rp2 : rp);
        jobs.add(lora->A[1], 1, r, H, true, fused ? At_gu + rp : At_gu + H * rp, 1, H, rp, fused ? rp2 : rp);
        if ((rc = launch_panel_prep(jobs, stream))) return rc;
    } else {
        (void)cv.take<bf16_t>(0);
    }
    bf16_t* dh = cv.take<bf16_t>(M * I * 2);
    bf16_t* dgu = cv.take<bf16_t>(M * 2 * I * 2);         // [M, 2I]: dgate | dup
    bf16_t* dx_u = cv.take<bf16_t>(M * H * 2);            // unfused dgrads: the up projection's share of dX
    bf16_t* v_d = cv.take<bf16_t>(M * (rp ? rp : 16) * 2);
    bf16_t* v_gu = cv.take<bf16_t>(M * (rp ? rp2 : 32) * 2);
    float* pair = cv.take<float>((int64_t)(rp ? rp2 : 32) * H * 4);
    float* part = cv.take<float>(0);
    const int64_t part_bytes = workspace_bytes - cv.used;
    bf16_t *dgate = dgu, *dup = dgu + I;

    // ---- down projection
    if (rp && (rc = launch_small_nt(dy, lddy, M, H, Bt_d, rp, s, v_d, nullptr, nullptr, 1, true, stream))) return rc;
    if ((rc = launch_tile_gemm(down, false, dy, lddy, M, nullptr, nullptr, rp ? v_d : nullptr, At_d, rp, nullptr, dh, I, stream, who, part, part_bytes))) return rc;
    if (rp) {
        if ((rc = launch_tn(dy, lddy, H, su_d, rp, r, M, false, grads->dB[2], part, nullptr, 1, stream))) return rc;       // [H, r]
        if ((rc = launch_tn(h, I, I, v_d, rp, r, M, true, grads->dA[2], part, nullptr, 1, stream))) return rc;             // [r, I]
    }
    // ---- SwiGLU, and s * dgate . B_g^T, s * dup . B_u^T: one pass over (gate, up, dh) where the rank allows, so that the
    // two products do not read dgate | dup back
    const int64_t ld_v = fused ? rp2 : rp;
    bf16_t* v_g = v_gu;
    bf16_t* v_u = fused ? v_gu + rp : v_gu + M * rp;
    const bool one_pass = rp && g_mlp_silu_nt && silu_bwd_nt_supported(I, rp);
    if (one_pass) {
        if ((rc = launch_silu_bwd_nt(gu, gu + I, 2 * I, dh, I, dgate, dup, 2 * I, M, I, Bt_g, Bt_u, rp, s, v_g, v_u, ld_v, stream))) return rc;
    } else if ((rc = xq_silu_mul_bwd(gu, gu + I, 2 * I, dh, I, nullptr, dgate, dup, 2 * I, nullptr, M, I, stream))) {
        return rc;
    }
    // ---- gate / up
    if (rp) {
        if (!one_pass) {
            if ((rc = launch_small_nt(dgate, 2 * I, M, I, Bt_g, rp, s, v_g, nullptr, nullptr, 1, true, stream, ld_v))) return rc;
            if ((rc = launch_small_nt(dup, 2 * I, M, I, Bt_u, rp, s, v_u, nullptr, nullptr, 1, true, stream, ld_v))) return rc;
        }
        const SuLayout sl = su_layout(saved->gate_up_fused == 1, rp, M);
        if ((rc = launch_tn(dgate, 2 * I, I, su_gu, rp, r, M, false, grads->dB[0], part, nullptr, 1, stream, nullptr, sl.pitch))) return rc;        // [I, r]
        if ((rc = launch_tn(dup, 2 * I, I, su_gu + sl.up_offset, rp, r, M, false, grads->dB[1], part, nullptr, 1, stream, nullptr, sl.pitch))) return rc;
        if (fused) {       // [2 rp, H] = [v_g | v_u]^T . x, then its two bands
            if ((rc = launch_tn(x, ldx, H, v_gu, rp2, rp2, M, true, pair, part, nullptr, 1, stream))) return rc;
            const unsigned blocks = (unsigned)xq_cdiv((int64_t)r * H, 256);
            copy_rows_kernel<<<dim3(blocks), 256, 0, stream>>>(pair, H, 0, r, grads->dA[0]);
            copy_rows_kernel<<<dim3(blocks), 256, 0, stream>>>(pair, H, rp, r, grads->dA[1]);
            XQ_CHECK_LAUNCH(who);
        } else {
            if ((rc = launch_tn(x, ldx, H, v_g, rp, r, M, true, grads->dA[0], part, nullptr, 1, stream))) return rc;       // [r, H]
            if ((rc = launch_tn(x, ldx, H, v_u, rp, r, M, true, grads->dA[1], part, nullptr, 1, stream))) return rc;
        }
    }
    if (!dx) return XQ_OK;
    if (fused) {
        const TwoBanks two{up, nullptr, nullptr};
        return launch_tile_gemm(gate, false, dgu, 2 * I, M, nullptr, nullptr, rp ? v_gu : nullptr, At_gu, rp2, nullptr, (bf16_t*)dx, lddx,
                                stream, who, nullptr, 0, &two);
    }
    if ((rc = launch_tile_gemm(gate, false, dgate, 2 * I, M, nullptr, nullptr, rp ? v_g : nullptr, At_gu, rp, nullptr, (bf16_t*)dx, lddx, stream, who, part, part_bytes))) return rc;
    if ((rc = launch_tile_gemm(up, false, dup, 2 * I, M, nullptr, nullptr, rp ? v_u : nullptr, At_gu + H * rp, rp, nullptr, dx_u, H, stream, who, part, part_bytes))) return rc;
    add_rows_kernel<<<dim3((unsigned)xq_cdiv(M * (H / 8), 256)), 256, 0, stream>>>((bf16_t*)dx, lddx, dx_u, H, M, H / 8);
    XQ_CHECK_LAUNCH(who);
    return XQ_OK;
}
