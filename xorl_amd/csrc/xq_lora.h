// Low-rank (LoRA) helper kernels: factor preparation, the skinny "down"
// products (x.A^T, dy.B) and the weight-gradient products (dy^T.u, v^T.x).
// All are HBM-bound: they stream one large bf16 activation matrix once.
#pragma once

#include "xq_common.h"

namespace xq {

// out[i][j] (bf16, [R_out, C_out], zero padded) = in[i][j] or in[j][i];  `in` is
// fp32 or bf16 with shape [R_in, C_in] per expert.
// up to three single-matrix conversions (same source dtype) done by one launch
struct FactorPrepJobs {
    const void* in[3];
    bf16_t* out[3];
    int64_t R_in[3], C_in[3], R_out[3], C_out[3];
    int transpose[3];
    int in_f32, n;
    void add(const void* src, int64_t r_in, int64_t c_in, bool tr, bf16_t* dst, int64_t r_out, int64_t c_out) {
        in[n] = src; out[n] = dst; R_in[n] = r_in; C_in[n] = c_in; R_out[n] = r_out; C_out[n] = c_out; transpose[n] = tr ? 1 : 0;
        ++n;
    }
};
int launch_factor_prep_multi(const FactorPrepJobs& jobs, hipStream_t stream);

// Every LoRA panel of a call in one launch: job k converts a [n_src, R_in, C_in] fp32 / bf16 factor (n_src = 1 or
// the expert count) into bf16 [n_out, R_out, C_out], optionally transposed, zero padded; n_src == 1 < n_out repeats
// the one source matrix for every expert (a factor shared by all experts, handed to a kernel that indexes panels
// by expert).  `pitch` (0: C_out) is the row length of the destination, for a panel that is a column band of a
// wider one; `e_stride` (0: R_out * pitch) the distance between two experts' panels in the destination, for a panel
// that is a row band of a taller one.
constexpr int MAX_PANEL_JOBS = 6;
struct PanelJobs {
    const void* in[MAX_PANEL_JOBS];
    bf16_t* out[MAX_PANEL_JOBS];
    int64_t R_in[MAX_PANEL_JOBS], C_in[MAX_PANEL_JOBS], R_out[MAX_PANEL_JOBS], C_out[MAX_PANEL_JOBS], pitch[MAX_PANEL_JOBS];
    int64_t e_stride[MAX_PANEL_JOBS];
    int32_t n_src[MAX_PANEL_JOBS], n_out[MAX_PANEL_JOBS], transpose[MAX_PANEL_JOBS];
    int32_t in_f32, n;
    bf16_t* add(const void* src, int n_src_, int64_t r_in, int64_t c_in, bool tr, bf16_t* dst, int n_out_, int64_t r_out,
                int64_t c_out, int64_t pitch_ = 0, int64_t e_stride_ = 0) {
        in[n] = src; out[n] = dst; R_in[n] = r_in; C_in[n] = c_in; R_out[n] = r_out; C_out[n] = c_out;
        pitch[n] = pitch_ ? pitch_ : c_out;
        e_stride[n] = e_stride_ ? e_stride_ : r_out * pitch[n];
        n_src[n] = n_src_; n_out[n] = n_out_; transpose[n] = tr ? 1 : 0;
        ++n;
        return dst;
    }
};
int launch_panel_prep(const PanelJobs& jobs, hipStream_t stream);
int launch_factor_prep(const void* in, int in_dtype, int64_t R_in, int64_t C_in, bool transpose,
                       bf16_t* out, int64_t R_out, int64_t C_out, int64_t num_experts, hipStream_t stream);

// T[rows, r_pad] = bf16(scale * In[rows, Kc] . F[r_pad, Kc]^T).
//   dense (offsets == NULL): rows = n_rows, one F;
//   grouped: rows in expert order, F[e] = F + e*r_pad*Kc (or shared).
int launch_small_nt(const bf16_t* In, int64_t ld_in, int64_t n_rows, int64_t Kc, const bf16_t* F,
                    int r_pad, float scale, bf16_t* T, const int32_t* offsets,
                    const int32_t* tile_offsets, int32_t num_experts, bool shared_f, hipStream_t stream,
                    int64_t ld_t = 0,       // row pitch of T in elements (0: r_pad), to write a column band of a wider matrix
                    bf16_t* T2 = nullptr, int split = 0,    // result columns from `split` on go to T2 (same pitch): two panels' products from one pass
                    const int32_t* row_map = nullptr,       // grouped: product row i is made from row row_map[i] of In, and the
                    bf16_t* copy_out = nullptr, int64_t ld_copy = 0);   // gathered rows are also written to copy_out [rows, Kc] (if given)

// SwiGLU backward and the two low-rank products of its outputs in one pass (r_pad 16 or 32): dgate | dup as
// xq_silu_mul_bwd writes them, Tg = scale * dgate . Fg^T, Tu = scale * dup . Fu^T as two
// launch_small_nt calls on them would (same bits)
bool silu_bwd_nt_supported(int64_t cols, int r_pad);
int launch_silu_bwd_nt(const bf16_t* gate, const bf16_t* up, int64_t ld_gu, const bf16_t* dh, int64_t ld_dh, bf16_t* dgate,
                       bf16_t* dup, int64_t ld_out, int64_t n_rows, int64_t cols, const bf16_t* Fg, const bf16_t* Fu, int r_pad,
                       float scale, bf16_t* Tg, bf16_t* Tu, int64_t ld_t, hipStream_t stream,
                       // routed rows in expert order (offsets != NULL): a factor pair per expert ([E][r_pad][cols]) unless
                       // shared, the rows' routing weights applied and (d_row_w != NULL) their gradients written
                       const int32_t* offsets = nullptr, const int32_t* tile_offsets = nullptr, int32_t num_experts = 1,
                       bool shared_fg = true, bool shared_fu = true, const float* row_w = nullptr, float* d_row_w = nullptr,
                       float swiglu_limit = 0.0f);     // > 0: the gate pre-activation is clamped to [-limit, limit], its gradient masked outside

// the forward in the same organisation: h = SwiGLU(gate, up) as xq_silu_mul_fwd writes it (routed rows: times the row's
// weight) and T = scale * h . F^T as launch_small_nt on h would (same bits)
int launch_silu_fwd_nt(const bf16_t* gate, const bf16_t* up, int64_t ld_gu, bf16_t* h, int64_t ld_h, int64_t n_rows, int64_t cols,
                       const bf16_t* F, int r_pad, float scale, bf16_t* T, int64_t ld_t, hipStream_t stream,
                       const int32_t* offsets = nullptr, const int32_t* tile_offsets = nullptr, int32_t num_experts = 1,
                       bool shared_f = true, const float* row_w = nullptr, float swiglu_limit = 0.0f);

// xq_silu_mul_fwd / xq_silu_mul_bwd with a SwiGLU limit on the gate pre-activation (ops/moe/triton.py:127-141; <= 0: none)
int silu_mul_fwd_limit(const void* gate, const void* up, int64_t ld_in, const float* row_w, void* h, int64_t ld_h, int64_t rows,
                       int64_t cols, float limit, void* stream);
int silu_mul_bwd_limit(const void* gate, const void* up, int64_t ld_in, const void* dh, int64_t ld_dh, const float* row_w, void* dgate,
                       void* dup, int64_t ld_out, float* d_row_w, int64_t rows, int64_t cols, float limit, void* stream);

// out[c][j] (or out[j][c] when transpose_out) = sum_m P[m][c] * Q[m][j], fp32.
//   dense: all rows, split over `splits` row ranges, partials in `partial`
//          ([splits][width][r_pad] fp32) reduced in fixed order (deterministic);
//   grouped: out[e] over rows [offsets[e], offsets[e+1]); zero for empty experts.
// r_out is the number of valid columns of Q (<= r_pad) written.
int64_t tn_partial_bytes(int64_t n_rows, int64_t width, int r_pad);
int launch_tn(const bf16_t* P, int64_t ldp, int64_t width, const bf16_t* Q, int r_pad, int r_out,
              int64_t n_rows, bool transpose_out, float* out, float* partial,
              const int32_t* offsets, int32_t num_experts, hipStream_t stream,
              const int32_t* row_limit = nullptr,    // dense form: contract only rows below *row_limit (device value)
              int64_t ldq = 0,                       // row pitch of Q in elements (0: r_pad), for a column band of a wider matrix
              const int32_t* p_rows = nullptr);      // optional: row m of the contraction is row p_rows[m] of P (Q rows stay in order)

int launch_zero_fill(void* p, int64_t bytes, hipStream_t stream);

// fused dequant-GEMM launcher (xq_gemm.hip).  `two`: a grouped launch over two block-fp8 banks of one shape -- the
// forward (contract_cols false) writes [rows, 2 * cols] with the second bank's columns, side term su2 / lora_right2,
// after the first's; the dgrad (contract_cols true) contracts A [rows, 2 * cols] against both banks into one sum.
struct TwoBanks {
    const xq_weight* w2;
    const bf16_t* su2;
    const bf16_t* lora_right2;
};
int64_t tile_gemm_partial_bytes(int64_t n_rows, int64_t Nout, int64_t Kc);   // split-K scratch a dense launch may want
bool two_banks_supported(const xq_weight* w);
bool two_dense_supported(const xq_weight* w);   // dense [N, K] pair: one dgrad launch, dX = [dY1 | dY2] . [W1 ; W2]
int launch_gate_up_swiglu(const xq_weight* wg, const xq_weight* wu, const bf16_t* x, int64_t ldx, int64_t M,
                          const bf16_t* su_g, const bf16_t* su_u, int64_t ld_su, const bf16_t* lr_g, const bf16_t* lr_u,
                          int r_pad, const bf16_t* bias_g, const bf16_t* bias_u, bf16_t* gu, int64_t ldgu, bf16_t* h,
                          int64_t ldh, hipStream_t stream);
int launch_tile_gemm(const xq_weight* w, bool contract_cols, const bf16_t* A, int64_t lda, int64_t n_rows,
                     const int32_t* offsets, const int32_t* tile_offsets, const bf16_t* su, const bf16_t* lora_right,
                     int r_pad, const bf16_t* bias, bf16_t* C, int64_t ldc, hipStream_t stream, const char* who,
                     float* partial, int64_t partial_bytes, const TwoBanks* two = nullptr,
                     const int32_t* a_rows = nullptr,    // grouped, optional: row i of the problem is row a_rows[i] of A,
                     int64_t a_span_rows = 0);           // ... which has this many rows (0: not known)
bool tile_gemm_takes_row_map(const xq_weight* w);        // ... which only the pipelined tile kernel does

int num_cus();   // compute units of the current device (xq_gemm.hip)

// skinny-M (M <= 64) forward path, xq_skinny.hip
bool skinny_supported(const xq_weight* w, int64_t M);
int64_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int r_pad);
int launch_skinny(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                  int lora_dtype, int r, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, void* workspace,
                  int64_t workspace_bytes, hipStream_t stream);

}  // namespace xq
