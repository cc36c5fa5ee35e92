/*
 * xq.h -- C ABI of libxq_hip.so: the MI355X (gfx950) implementation of xorl's
 * QLoRA quantized base-linear hot path.
 *
 * The reference (togethercomputer/xorl) has no FFI for this path: every
 * kernel is a Triton function called from Python.  Each entry point below
 * therefore names the Python function(s) of the reference it replaces
 * (paths relative to the xorl checkout).  A maintainer binds these with
 * ctypes (xorl_amd/_C.py holds every signature); no torch type appears in any signature.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless stated otherwise;
 *   - `stream` is a hipStream_t passed as void* (0 = the null stream);
 *   - the library allocates nothing: outputs and workspaces are the caller's;
 *   - every function validates its arguments on the host and returns
 *     XQ_OK (0) or a negative error code before launching anything;
 *     xq_last_error() returns a message for the calling thread's last error;
 *   - activations are bf16 row-major with an explicit row stride in elements.
 */
#ifndef XQ_H
#define XQ_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define XQ_OK 0
#define XQ_ERR_ARG (-1)      /* bad argument (shape, alignment, enum, null) */
#define XQ_ERR_UNSUPPORTED (-2)
#define XQ_ERR_LAUNCH (-3)   /* hipGetLastError() after a launch was not hipSuccess */

/* weight formats */
#define XQ_FMT_INT4 0   /* 4-bit offset-binary codes, w = (nib - 8) * scale            */
#define XQ_FMT_NVFP4 1  /* e2m1 codes, per-16 block scale * fp32 global scale          */
#define XQ_FMT_FP8 2    /* e4m3fn bytes, fp32 scale per 128x128 block                  */
#define XQ_FMT_NF4 3    /* NormalFloat4 codes, w = level[nib] * scale (fp32/bf16 scale) */

/* storage layouts of the 4-bit formats (fp8 is symmetric: layout is ignored)
 *   FLAT: decoded shape [rows, cols]; nibble pairs and scale groups run along
 *         cols; packed [rows, cols/2], scales [rows, cols/group].  This is the
 *         dense module's [out_features, in_features] storage.
 *   GKN : decoded shape [rows, cols]; nibble pairs and scale groups run along
 *         rows; packed [rows/2, cols], scales [rows/group, cols].  This is the
 *         expert bank's [in_features, out_features] storage.                 */
#define XQ_LAYOUT_FLAT 0
#define XQ_LAYOUT_GKN 1

/* scale element types */
#define XQ_SCALE_F32 0
#define XQ_SCALE_BF16 1
#define XQ_SCALE_E4M3 2

/* element types of outputs / LoRA factors */
#define XQ_DT_BF16 0
#define XQ_DT_F32 1

/* A bank of `num_experts` equally shaped quantized matrices (1 for a dense
 * linear).  Expert e starts at packed + e*packed_bytes, scales + e*scale_bytes
 * (both derived from the shape), global_scale[e]. */
typedef struct xq_weight {
    int32_t format;       /* XQ_FMT_*    */
    int32_t layout;       /* XQ_LAYOUT_* */
    int32_t scale_dtype;  /* XQ_SCALE_*  */
    int32_t group;        /* int4 / nf4: any even divisor of the grouped dim (128 / 64 typical); nvfp4: 16; fp8: 128 */
    int64_t rows;         /* decoded rows */
    int64_t cols;         /* decoded cols */
    int32_t num_experts;
    int32_t reserved;
    const void* packed;
    const void* scales;
    const float* global_scale; /* nvfp4 only: num_experts floats; else NULL */
} xq_weight;

/* ---- library ---------------------------------------------------------- */
const char* xq_version(void);
const char* xq_last_error(void);

/* Per-launch timing of the fused dequant-GEMM kernel (the dominant kernel)
 * with HIP events on the launch stream; used by the benchmark's roofline
 * figure.  No counterpart in the reference.  xq_profile_enable(1) starts
 * recording (at most 8192 launches), xq_profile_collect waits for the
 * recorded launches and returns their count, summed duration and summed
 * algorithmic FLOPs (2*rows*Nout*(Kc + r_pad) each), then resets. */
int xq_profile_enable(int on);
int xq_profile_collect(int* n_launches, double* total_ms, double* total_flops);

/* A plain streaming read of `bytes` bytes (a multiple of 16, 16-byte
 * aligned) that does nothing else; `out` is one device word it practically
 * never writes.  For the benchmark: timed next to the weight-streaming
 * forwards it gives the measured ceiling for a read of that size.  No
 * counterpart in the reference. */
int xq_read_probe(const void* data, int64_t bytes, uint32_t* out, void* stream);

/* Kernel selection of the fused dequant-GEMM entry points (dense and grouped),
 * for tests and A/B measurements; no counterpart in the reference.
 *   0 (default): by problem size.  Block-fp8 and FLAT int4/nvfp4 weights with a
 *      power-of-two group >= 16 use the pipelined tile kernel, with 256x256 tiles
 *      when those fill the chip and 128x128 tiles otherwise; other weights (GKN
 *      4-bit banks, odd groups) use the generic single-buffered 128x128 kernel;
 *   1: always the generic kernel;
 *   2 / 3: the pipelined kernel with 256x256 / 128x128 tiles whenever the format
 *      allows it, whatever the size. */
int xq_set_tile_policy(int policy);

/* The 256x256 tile kernel (unsplit launches) is a persistent program: one block per compute unit walks the
 * tiles b, b + grid, ... and requests its next tile's first operands before it stores the finished tile.
 * enabled = 0 launches one block per tile instead -- the same kernel and, bit for bit, the same results; a
 * process-wide switch for tests and A/B measurements (XQ_PERSIST=0 in the environment sets it at load time);
 * no counterpart in the reference. */
int xq_set_persistent_tiles(int enabled);

/* Dense block-fp8 products on 256 x 256 tiles (forward, dgrad; unsplit) run on the kernel that loads both operand tiles
 * straight into LDS, keeps the weight tile as e4m3 bytes there and multiplies with v_mfma_f32_16x16x32_bf16 (enabled = 1,
 * the default), or on the tile kernel that every other format and the expert banks use (enabled = 0).  Both decode to the
 * reference's bf16 values bit for bit; their sums run in different orders, so outputs agree to rounding.  A process-wide
 * switch for tests and A/B measurements (XQ_FP8_DIRECT in the environment sets it at load time); no counterpart in the
 * reference. */
int xq_set_fp8_direct_tiles(int enabled);

/* xq_mlp_fwd on block-fp8 weights runs gate and up either as two launches followed by one pass that writes h = SwiGLU and
 * forms the down projection's low-rank intermediate on the way (enabled = 0, the default), or as ONE launch over both weights
 * with the SwiGLU in its epilogue (enabled = 1).  Same outputs and saved activations bit for bit when the plain launches run on
 * the same tile kernel (xq_set_fp8_direct_tiles(0)), to rounding otherwise (other summation order); the saved low-rank
 * intermediates of gate and up are laid out differently, which xq_mlp_saved::gate_up_fused records for the backward: the
 * switch is only the default of a forward whose struct does not say (a negative field) and may change at any time.
 * A process-wide switch for tests and A/B measurements (XQ_MLP_GU in the environment sets it at load time); no counterpart
 * in the reference. */
int xq_set_mlp_gate_up_fused(int enabled);
int xq_get_mlp_gate_up_fused(void);   /* the current default: 0 or 1 */

/* xq_linear_fwd with M <= 16 rows runs as ONE launch where the shape and the LoRA operands allow it (FLAT weight,
 * K % 512 == 0 for block_fp8 / K % 1024 == 0 for the 4-bit formats, K <= 12288; fp32 factors with r <= 16, r % 4 == 0,
 * 16-byte aligned): whole weight rows per block, the low-rank intermediate formed once per launch and passed between
 * blocks through device memory that belongs to the library (tied to the call's workspace pointer: calls with different
 * workspaces may overlap on a device as before).  enabled = 0 keeps every M <= 64 forward on the two-launch
 * organisation (K split over blocks + epilogue); results of the two agree to rounding, not bit for bit (different
 * summation orders).  A process-wide switch for tests and A/B measurements (XQ_SKINNY_ROWS=0 in the environment sets
 * it at load time); no counterpart in the reference. */
int xq_set_skinny_one_launch(int enabled);
/* One token (M = 1) against a FLAT block-fp8, nvfp4 (e4m3 block scales), nf4 (groups of 64) or int4 weight whose rows are whole KBs
 * (in_features % 1024 == 0, the 4-bit formats: % 2048; at most 15 KB per row; int4 only on shapes on which it is the
 * faster kernel -- at most 4096 rows, or rows of 8192 elements and more) runs a kernel of its own inside the one-launch
 * path: no matrix cores, waves that stream whole rows (block fp8: the rate of a plain read from HBM), same slots and same
 * failure rules.  enabled = 0 sends those forwards to the kernel of the larger row counts (results agree to rounding: same
 * decoded values, other summation order).  Process-wide switch for tests and A/B measurements (XQ_SKINNY_GEMV=0 in the
 * environment); no counterpart in the reference. */
int xq_set_skinny_gemv(int enabled);

/* Test switch (process-wide, no counterpart in the reference): how many times a bounded wait of the one-launch skinny
 * kernel looks before it gives up (limit <= 0 restores the default, about a second of waiting).  The waits are for other
 * blocks of the same launch (the published parts of x . A^T; the count of blocks that have read the launch count).  A
 * block whose wait gives up writes NaN to its outputs and ends like every other block; if it is the block that closes the
 * launch it marks the library's slot for this workspace failed, and every later forward through that slot writes NaN
 * (never values made from another launch's sums) until xq_skinny_reset().  A small limit forces those paths from the host
 * without any kernel hanging or faulting. */
int xq_set_skinny_spin_limit(int limit);
/* Clears the library's slots on the current device (launch counts, failure marks, published parts).  Synchronises the
 * device before and after: call it with no forward in flight.  No counterpart in the reference. */
int xq_skinny_reset(void);
/* What the one-launch skinny forwards on the current device have reported since the last call.  *gave_up: blocks whose
 * bounded wait gave up (each wrote NaN to its outputs); *failed_slots: slots marked failed (every forward through such a
 * slot writes NaN).  Either pointer may be NULL.  The call waits for `stream`, reads a few words back and, if anything was
 * found, waits for the whole device and clears the marks and the count, so that later forwards are exact again: a host
 * calls it where it waits for results anyway (before it reads sampled tokens, say) and treats a non-zero report as "the
 * forwards since the last call may hold NaN".  The slots are a fixed pool (256 per device) keyed by workspace pointer: a
 * slot that a HIP-graph capture recorded stays with its workspace for good, another one changes hands only after the
 * stream of its last launch has run dry, and a forward that can get no slot runs the two-launch organisation instead.
 * No counterpart in the reference. */
int xq_skinny_status(int* gave_up, int* failed_slots, void* stream);

/* ---- decode ------------------------------------------------------------
 * out[e] = decoded weight of expert e, shape [rows, cols], bf16 or fp32.
 * Replaces int4_dequantize / int4_dequantize_gkn
 *   (ops/quantize/int4_quantize.py:113-127, int4_gkn_quantize.py:176-216),
 * nvfp4_dequantize / nvfp4_dequantize_gkn
 *   (ops/quantize/nvfp4_quantize.py:157-177, nvfp4_gkn_quantize.py:238-273),
 * nf4_dequantize / nf4_dequantize_gkn
 *   (ops/quantize/nf4_quantize.py:154-185, nf4_gkn_quantize.py:182-, levels nf4_codec.py:18-35),
 * block_fp8_dequantize_gkn (ops/quantize/block_fp8_gkn_quantize.py:157-180;
 *   XQ_DT_F32 gives that function's fp32 output, XQ_DT_BF16 gives the
 *   `.to(bf16)` its callers apply, qlora/modules/linear.py:373).
 * Bit-exact with the reference arithmetic. */
int xq_decode(const xq_weight* w, void* out, int out_dtype, void* stream);

/* ---- dense QLoRA linear -------------------------------------------------
 * Replaces QLoRALinear.forward (qlora/modules/linear.py:369-385) and its
 * autograd backward.  The weight is FLAT [N, K]. */

/* Bytes of scratch the dense entry points need for (M, N, K, r): the prepared
 * LoRA panels and partial sums of the factor gradients (r > 0) and, for row
 * counts that leave most of the chip without a tile, the fp32 partial sums of
 * the split-K product.  With r == 0 the workspace is optional: a call without
 * it (or with fewer bytes) runs the product unsplit. */
int64_t xq_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int r);

/* y[M,N] = x[M,K] . deq(W)^T + bias + s * (x . A^T) . B^T      (bf16 out)
 *   lora_A [r,K], lora_B [N,r] in lora_dtype (fp32 or bf16), r in {0..64};
 *   su_out (optional, bf16 [M, r_pad], r_pad = r rounded up to 16) receives
 *   bf16(s * x . A^T) for reuse by xq_linear_bwd; with su_out == NULL and
 *   M <= 64 (K % 128 == 0) the weight-streaming skinny kernel is used;
 *   workspace: xq_linear_workspace_bytes(...) bytes, 256-byte aligned. */
int xq_linear_fwd(const xq_weight* w, const void* x, int64_t ldx, int64_t M,
                  const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                  const void* bias_bf16, void* y, int64_t ldy, void* su_out,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* h[M, I] = silu(gate) * up for a weight that holds gate | up stacked, W [2 I, K] (one QLoRA linear: the reference's
 * default gate_up_proj module, qlora/utils.py:33-37, followed by fused_silu_and_mul, ops/fused_silu_and_mul.py:22-60;
 * call site models/transformers/qwen3/modeling_qwen3.py:62-70): the forward of xq_linear_fwd on all 2 I rows and the
 * SwiGLU arithmetic of xq_silu_mul_fwd on its rounded outputs (same rounding points, bit-identical to the two calls).
 * For M <= 16, where the weight takes the one-launch skinny kernel in two rounds (I % 48 == 0, K <= 4096 at one byte
 * per weight), one launch: a block holds the gate rows and the up rows of its columns and writes h directly.
 * Otherwise the two calls run one after the other inside this one (gate | up goes through the workspace).
 * workspace: xq_linear_fwd_swiglu_workspace_bytes(M, 2 I, K, r) bytes, 256-byte aligned. */
int64_t xq_linear_fwd_swiglu_workspace_bytes(int64_t M, int64_t N2, int64_t K, int r);
int xq_linear_fwd_swiglu(const xq_weight* w, const void* x, int64_t ldx, int64_t M,
                         const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                         const void* bias_bf16, void* h, int64_t ldh, void* workspace, int64_t workspace_bytes, void* stream);

/* Several forwards that share x: y_i = x . deq(W_i)^T + bias_i + s_i * (x . A_i^T) . B_i^T, i < n_jobs <= 4.
 * Replaces the separate module calls of the reference's attention and MLP blocks
 * on one input (q_proj / k_proj / v_proj: src/xorl/models/layers/attention/multi_head_attention.py:93-95;
 * gate_proj / up_proj: src/xorl/models/transformers/qwen3/modeling_qwen3.py:75-76) when a model keeps them as
 * separate modules (unfuse_for_tp); each forward is the one of qlora/modules/linear.py:369-385.
 * All weights contract over the same K.  For M <= 16, with weights of one
 * format that fit the one-launch skinny kernel, all forwards run as ONE launch
 * (the grid holds each forward's blocks one after the other); otherwise they run
 * one after the other as xq_linear_fwd(..., su_out = NULL).  Results are
 * bit-identical to separate xq_linear_fwd calls either way.
 * workspace: xq_linear_fwd_multi_workspace_bytes(...) bytes, 256-byte aligned. */
#define XQ_LINEAR_MULTI_MAX 4
typedef struct xq_linear_job {
    const xq_weight* w;
    const void* lora_A;     /* [r, K] in lora_dtype */
    const void* lora_B;     /* [N, r] in lora_dtype */
    int32_t r;              /* 0 .. 64 */
    float scaling;
    const void* bias_bf16;  /* [N] or NULL */
    void* y;                /* bf16 [M, N], row stride ldy */
    int64_t ldy;
} xq_linear_job;
int64_t xq_linear_fwd_multi_workspace_bytes(const xq_linear_job* jobs, int n_jobs, int64_t M);
int xq_linear_fwd_multi(const xq_linear_job* jobs, int n_jobs, const void* x, int64_t ldx, int64_t M, int lora_dtype,
                        void* workspace, int64_t workspace_bytes, void* stream);

/* xq_linear_fwd for callers that cannot allocate device memory or be handed a
 * workspace: code under HIP-graph capture, tight rollout / serving loops,
 * harnesses that forbid allocation.  No counterpart in the reference (its
 * forward allocates through torch).  Same arguments and results as
 * xq_linear_fwd with su_out == NULL (bit-identical: the same kernels run), but
 * the scratch is a buffer of XQ_STATIC_SCRATCH_BYTES built into the library's
 * code object, one copy per device, resolved once per device at the first call
 * made with that device current.  The call allocates and frees nothing.
 * Shapes whose xq_linear_workspace_bytes(M, N, K, r) exceeds the buffer are
 * rejected with XQ_ERR_ARG.  All calls on one device share that device's
 * buffer: calls that overlap in time on one device (two streams, two host
 * threads) race; calls on one stream, or ordered by events, do not.  Nothing in
 * the buffer has to start at zero, so nothing is cleared between calls. */
#define XQ_STATIC_SCRATCH_BYTES (32ll << 20)
int64_t xq_static_scratch_bytes(void);
int xq_linear_fwd_static(const xq_weight* w, const void* x, int64_t ldx, int64_t M,
                         const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                         const void* bias_bf16, void* y, int64_t ldy, void* stream);

/* dx[M,K] = dy . deq(W) + s * (dy . B) . A   (bf16)
 * dA[r,K] = s * (dy . B)^T . x               (fp32, overwritten)
 * dB[N,r] = s * dy^T . (x . A^T)             (fp32, overwritten)
 *   su: the buffer xq_linear_fwd wrote (or NULL: recomputed from x);
 *   any of dx / dA / dB may be NULL to skip it. */
int xq_linear_bwd(const xq_weight* w, const void* x, int64_t ldx, const void* dy, int64_t lddy,
                  int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                  float scaling, const void* su, void* dx, int64_t lddx, float* dA, float* dB,
                  void* workspace, int64_t workspace_bytes, void* stream);

/* ---- merging the LoRA update into the base weight ------------------------
 * W'[n,k] = deq(W)[n,k] + scaling * sum_j B[n,j] * A[j,k], W FLAT [N, K]
 * (in_features % 16 == 0), factors fp32 or bf16, r in {0..64}; the low-rank
 * product is evaluated to ~16 significant bits per factor (hi/lo bf16 split).
 *
 * xq_merge_dense writes W' as bf16 or fp32 [N, K] without materialising
 * deq(W).  bf16: bf16(bf16(deq) + bf16(delta)), the arithmetic of the
 * reference's weight-sync merge (server/weight_sync/handler.py:2119-2131:
 * `_dequantize_weight().to(bf16) + get_delta_weight().to(bf16)`).  fp32: the
 * sum merge_weights forms before it re-quantises (qlora/modules/
 * block_fp8_linear.py:111-115; for the 4-bit formats, whose decoders return
 * bf16, the bf16 sum widened to fp32).
 *
 * xq_merge_requant_fp8 (block_fp8 only) is merge_weights + _quantize_and_store
 * in one pass (block_fp8_linear.py:111-119 with block_fp8_quantize_gkn,
 * ops/quantize/block_fp8_gkn_quantize.py:40-121): per 128x128 block
 * s = max(amax(W') / 448, 1e-12), bytes = e4m3(clamp(W' / s, +-448)).
 * packed_out / scales_out may be the weight's own buffers (in-place).
 *
 * Both take a workspace of xq_merge_workspace_bytes(N, K, r) bytes (256-byte
 * aligned; may be NULL when r == 0): the factors are split once per call
 * into bf16 hi/lo panels there. */
int64_t xq_merge_workspace_bytes(int64_t N, int64_t K, int r);
int xq_merge_dense(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                   float scaling, void* out, int out_dtype, void* workspace, int64_t workspace_bytes,
                   void* stream);
int xq_merge_requant_fp8(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                         float scaling, void* packed_out, float* scales_out, void* workspace,
                         int64_t workspace_bytes, void* stream);

/* nvfp4 counterpart, in two launches because the scales hang on a tensor-wide
 * quantity (qlora/modules/nvfp4_linear.py:126-139 with nvfp4_quantize,
 * ops/quantize/nvfp4_quantize.py:25-60,102-154).  The merged values are those
 * xq_merge_dense writes as bf16.
 *   xq_merge_amax: amax_out[0] = max |W'| over the matrix (any format), which
 *     the module blends into its running amax (`_ema_amax.lerp_`).
 *   xq_merge_requant_nvfp4: with global_amax[0] (device memory) as the tensor
 *     amax, per 16-element block: codes = e2m1(clamp(W' * (6 / amax_b), +-6)),
 *     block scale = e4m3(amax_b / global_amax * 448); global_scale_out[0] =
 *     global_amax / 6 / 448.  codes_out [N, K/2] and block_scales_out
 *     [N, K/16] may be the weight's own buffers when its block scales are stored
 *     as e4m3; global_scale_out must be other memory than w->global_scale. */
int xq_merge_amax(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r, float scaling,
                  float* amax_out, void* workspace, int64_t workspace_bytes, void* stream);
int xq_merge_requant_nvfp4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                           float scaling, const float* global_amax, void* codes_out, void* block_scales_out,
                           float* global_scale_out, void* workspace, int64_t workspace_bytes, void* stream);

/* NF4 counterpart (qlora/modules/nf4_linear.py merge_weights with nf4_quantize,
 * ops/quantize/nf4_quantize.py:20-56): one pass; per 64-element group
 * scale = max(absmax, 1e-12) (fp32), code = nearest-level code of
 * clamp(W' / scale, +-1) by the midpoint rule.  The weight must hold fp32
 * scales per 64 elements; in_features % 64 == 0.  codes_out [N, K/2] and
 * scales_out [N*K/64] may be the weight's own buffers. */
int xq_merge_requant_nf4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                         float scaling, void* codes_out, float* scales_out, void* workspace,
                         int64_t workspace_bytes, void* stream);

/* int4 counterpart for a flat int4 weight with 128-element groups
 * (in_features % 128 == 0): W' = bf16(bf16(deq(W)) + bf16(delta)) as
 * xq_merge_dense forms it, re-encoded per group in the same pass.
 * symmetric = 0: the rule of ops/quantize/int4_quantize.py:12-41
 * (scale = max(absmax, 1e-12) * 2/15 in fp32, code = clamp(trunc(x * (1 /
 * scale) + 8.5), 0, 15)), scales_out fp32 [N, K/128].  symmetric = 1: scale =
 * bf16(absmax / 7), code = clamp(rne(x / scale), -7, 7) + 8, scales_out bf16
 * [N, K/128] -- the rule of the int4 benchmark workload, which the reference
 * has no module for.  codes_out [N, K/2] and scales_out may be the weight's
 * own buffers when the scale type stays the same. */
int xq_merge_requant_int4(const xq_weight* w, const void* lora_A, const void* lora_B, int lora_dtype, int r,
                          float scaling, int symmetric, void* codes_out, void* scales_out, void* workspace,
                          int64_t workspace_bytes, void* stream);

/* ---- SwiGLU between gate/up and down ------------------------------------
 * Replaces fused_silu_and_mul (ops/fused_silu_and_mul.py:22-60 and its
 * backward): h = bf16(silu_fp32(gate)) * up, two roundings.  With row_w
 * (fp32 [rows], the routing weight of each expert-ordered row) it is the
 * routed form of ops/moe/lora.py:639-647, h = bf16(bf16(bf16(silu(g))*u)*w),
 * and the backward also returns d_row_w[row] = sum_c dh * bf16(bf16(silu(g))*u)
 * (ops/moe/lora.py:855-917).  row_w / d_row_w may be NULL. */
int xq_silu_mul_fwd(const void* gate, const void* up, int64_t ld_in, const float* row_w, void* h,
                    int64_t ld_h, int64_t rows, int64_t cols, void* stream);
int xq_silu_mul_bwd(const void* gate, const void* up, int64_t ld_in, const void* dh, int64_t ld_dh,
                    const float* row_w, void* dgate, void* dup, int64_t ld_out, float* d_row_w,
                    int64_t rows, int64_t cols, void* stream);

/* ---- grouped / routed (MoE experts) --------------------------------------
 * xq_route_build replaces the dispatch part of _MoeExpertsLoRAFunction.forward
 * (ops/moe/lora.py:579-583): expert_histogram, stable argsort by expert id,
 * cumsum.  selected [T*topk] int32 expert ids (row-major [T, topk]).
 * Outputs: counts [E], offsets [E+1] (exclusive prefix), scatter_index
 * [T*topk] (row in expert order of routed copy i), tile_offsets [2*(E+1)]:
 * two row-tile schedules of the grouped kernels back to back, the prefix of
 * ceil(count/128) in [0, E] and the prefix of ceil(count/256) in [E+1, 2E+1].
 * Deterministic and stable.  workspace: xq_route_workspace_bytes() bytes. */
int64_t xq_route_workspace_bytes(int64_t n_routed, int32_t num_experts);
int xq_route_build(const int32_t* selected, int64_t n_routed, int32_t num_experts,
                   int32_t* counts, int32_t* offsets, int32_t* scatter_index,
                   int32_t* tile_offsets, void* workspace, int64_t workspace_bytes, void* stream);

/* An expert id outside [0, num_experts) (the reference asserts on these on the device) drops that routed copy:
 * it is not counted, gets scatter_index -1, and the row movers below skip it -- xq_moe_scatter stores nothing for
 * it, xq_moe_gather adds nothing, xq_moe_scatter_scalar skips it, xq_moe_gather_scalar returns 0.  offsets[E] is
 * then smaller than n_routed and the rows [offsets[E], n_routed) of expert-ordered buffers belong to no expert. */
/* rows_out[scatter_index[i]] = rows_in[i / topk]   (moe_scatter, group_gemm/kernel/moe.py:266-312) */
int xq_moe_scatter(const void* in, int64_t ld_in, const int32_t* scatter_index, int64_t n_routed,
                   int32_t topk, int64_t width, void* out, int64_t ld_out, void* stream);
/* out[t] = sum_j rows[scatter_index[t*topk+j]] (+ rows2[...]), fp32 accumulate
 * (moe_gather / moe_add_gather, group_gemm/kernel/moe.py:102-141, :178-223) */
int xq_moe_gather(const void* rows, const void* rows2, int64_t ld_rows, const int32_t* scatter_index,
                  int64_t n_tokens, int32_t topk, int64_t width, void* out, int64_t ld_out, void* stream);
/* dst[scatter_index[i]] = float(src[i]) and dst[i] = src[scatter_index[i]]:
 * the routing-weight permutation of ops/moe/lora.py:644-646 and :857-858. */
int xq_moe_scatter_scalar(const void* src, int src_dtype, const int32_t* scatter_index, int64_t n,
                          float* dst, void* stream);
int xq_moe_gather_scalar(const float* src, const int32_t* scatter_index, int64_t n, void* dst,
                         int dst_dtype, void* stream);

/* Grouped projection over rows already in expert order:
 *   for each expert e with rows [offsets[e], offsets[e+1]):
 *     y[rows] = a[rows] . op(deq(W[e])) + su[rows] . Lr[e]^T
 * The bank is GKN [E, K_in, N_out]; transpose_w = 0 contracts over the bank's
 * rows (forward: y = x . W), 1 over its cols (dgrad: dx = dy . W^T).
 * su bf16 [R, r_pad] (already scaled) and lora_right bf16 [E, n_out, r_pad]
 * are the low-rank side term (NULL for none).
 * Replaces group_gemm_same_nk on dequantized banks
 * (ops/group_gemm/kernel/group_gemm.py:171-256) fused with
 * dequantize_all_experts (qlora/modules/moe_experts.py:486-498). */
int xq_grouped_gemm(const xq_weight* w, int transpose_w, const void* a, int64_t lda,
                    int64_t n_rows, const int32_t* offsets, const int32_t* tile_offsets,
                    const void* su, const void* lora_right, int r_pad,
                    void* y, int64_t ldy, void* stream);

/* out[e][i][j] (bf16, zero padded to [rows_out, cols_out]) = in[e][i][j] or
 * in[e][j][i]: brings fp32/bf16 LoRA factors into the bf16 operand layouts
 * the kernels above consume (the `.to(compute_dtype)` of ops/moe/lora.py:557-564). */
int xq_factor_prep(const void* in, int in_dtype, int64_t rows_in, int64_t cols_in, int transpose,
                   void* out_bf16, int64_t rows_out, int64_t cols_out, int64_t num_experts, void* stream);

/* Grouped low-rank helpers (bf16 in, fp32 accumulate):
 *   xq_grouped_lora_down: t[rows of e] = bf16(scale * a[rows of e] . F[e]^T),
 *       F bf16 [E, r_pad, K] (or one shared [r_pad, K]); t is [R, r_pad].
 *   xq_grouped_lora_wgrad: out[e] = P[rows of e]^T . Q[rows of e], fp32
 *       [E, p_width, r_out] (or [E, r_out, p_width] with transpose_out); zero
 *       for empty experts.  With offsets == NULL it is the dense form over all
 *       n_rows (one output; also the gradient of a factor shared by all
 *       experts).  Both forms split the rows over blocks and add the pieces in
 *       a fixed order (deterministic), in xq_lora_wgrad_workspace_bytes() bytes
 *       of scratch (256-byte aligned, required).  row_limit (device, may be NULL) restricts the dense form to
 *       the rows below *row_limit: offsets + E of xq_route_build, so that rows no expert owns (routed
 *       copies whose expert id was out of range) are left out.
 * Replace the small group_gemm_same_nk / group_gemm_same_mn calls of
 * ops/moe/lora.py:601-660 and :781-960. */
int xq_grouped_lora_down(const void* a, int64_t lda, int64_t n_rows, const int32_t* offsets,
                         const int32_t* tile_offsets, int32_t num_experts, const void* F, int shared,
                         int r_pad, int64_t K, float scale, void* t, void* stream);
int64_t xq_lora_wgrad_workspace_bytes(int64_t n_rows, int64_t width, int r_pad);
int xq_grouped_lora_wgrad(const void* P, int64_t ldp, int64_t p_width, const void* Q, int r_pad,
                          int r_out, int64_t n_rows, const int32_t* offsets, int32_t num_experts,
                          int transpose_out, float* out, void* workspace, const int32_t* row_limit, void* stream);

/* ---- the routed expert MLP in two calls ------------------------------------
 * xq_grouped_fwd / xq_grouped_bwd run the whole program of the reference's local LoRA expert compute
 * (_MoeExpertsLoRAFunction.forward / .backward, ops/moe/lora.py:525-713 and :715-1007; registry entry
 * MOE_EXPERT_BACKENDS_LORA, models/layers/moe/backend/__init__.py:421-445) on packed banks, composed from the entry
 * points above on the caller's stream: route build, scatter, gate / up projections with LoRA, SwiGLU with the
 * routing weight applied before the down projection, down projection with LoRA, top-k gather-sum; and its
 * backward (dX, routing-weight gradients, the six factor gradients; the frozen banks get none).  A host without
 * Python gets the routed MLP from these two calls.
 *
 * Banks are GKN: gate and up [E, H, I], down [E, I, H] (H, I multiples of 64).  LoRA factors in GKN form,
 * A[p] [A_experts[p], in, r] and B[p] [B_experts[p], r, out] for p = 0 gate, 1 up, 2 down, each held once
 * (shared by all experts: 1) or per expert (E); fp32 or bf16; r in 1..64.
 *
 * xq_grouped_saved names caller buffers the forward fills and the backward reads (R = n_tokens * topk routed
 * rows, r_pad = r rounded up to 16): xs bf16 [R, H] (token rows in expert order), gate_up bf16 [R, 2 I] (the
 * gate projection in columns [0, I), the up projection in [I, 2 I)), h bf16 [R, I], w_row fp32 [R], su_gate / su_up / su_down bf16 [R, r_pad], scatter_index int32 [R], offsets int32
 * [E + 1], tile_offsets int32 [2 (E + 1)], counts int32 [E].  A forward-only caller passes scratch for them.
 * xs may be NULL where xq_grouped_in_place(gate, up, down) returns 1 (banks that run on the pipelined tile kernel) and
 * the rows of hidden are 16-byte aligned: the routed rows are rows of hidden, each topk times, so the forward then
 * writes no expert-ordered copy of them and reads hidden through the routing instead; the backward of such a forward
 * is given the same hidden states as x_tokens (row stride ld_x_tokens, in elements) -- R * H * 2 bytes less to keep
 * per layer.  (The backward treats dy the same way whatever xs is.)
 * Factor gradients are fp32, shaped like the factors, overwritten (exact zeros for experts without rows).
 * hidden, out, dy, dx are bf16 [n_tokens, H] with row strides in elements; routing_w [n_tokens, topk] fp32 or
 * bf16, selected int32 [n_tokens, topk]; dx / d_routing may be NULL.  Expert ids outside [0, E) drop their copy.
 * workspace: xq_grouped_workspace_bytes(..., backward) bytes, 256-byte aligned. */
typedef struct xq_grouped_lora {
    const void* A[3];
    const void* B[3];
    int32_t A_experts[3];
    int32_t B_experts[3];
    int32_t dtype;      /* XQ_DT_* of all six factors */
    int32_t r;
    float scaling;
    /* > 0: the gate pre-activation is clamped to [-swiglu_limit, swiglu_limit] before the SiLU, and the gate gradient is zero
     * where the unclamped value lies outside that range (the swiglu_limit argument of the reference's expert functions,
     * ops/moe/lora.py:545-547,638,863,917-919; ops/moe/triton.py:127-141).  0: no clamp. */
    float swiglu_limit;
} xq_grouped_lora;

typedef struct xq_grouped_saved {
    void* xs;
    void* gate_up;
    void* h;
    float* w_row;
    void* su_gate;
    void* su_up;
    void* su_down;
    int32_t* scatter_index;
    int32_t* offsets;
    int32_t* tile_offsets;
    int32_t* counts;
    const void* x_tokens;      /* backward, when xs is NULL: the forward's hidden [n_tokens, H] bf16 */
    int64_t ld_x_tokens;
} xq_grouped_saved;

typedef struct xq_grouped_grads {
    float* dA[3];
    float* dB[3];
} xq_grouped_grads;

int64_t xq_grouped_workspace_bytes(int64_t n_tokens, int32_t topk, int32_t num_experts, int64_t hidden,
                                   int64_t intermediate, int r, int backward);
int xq_grouped_in_place(const xq_weight* gate, const xq_weight* up, const xq_weight* down);
int xq_grouped_fwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                   const void* hidden, int64_t ld_hidden, int64_t n_tokens, const void* routing_w, int rw_dtype,
                   const int32_t* selected, int32_t topk, void* out, int64_t ld_out,
                   const xq_grouped_saved* saved, void* workspace, int64_t workspace_bytes, void* stream);
int xq_grouped_bwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                   const void* dy, int64_t ld_dy, int64_t n_tokens, int32_t topk, const xq_grouped_saved* saved,
                   void* dx, int64_t ld_dx, void* d_routing, int rw_dtype, const xq_grouped_grads* grads,
                   void* workspace, int64_t workspace_bytes, void* stream);

/* The same forward for a handful of tokens with nothing kept for a backward (decode, rollout: the reference runs
 * _MoeExpertsLoRAFunction.forward, ops/moe/lora.py:525-713, under no_grad for these too, through the same grouped
 * GEMMs).  Same arguments as xq_grouped_fwd without `saved`, same result up to the summation order inside a dot
 * product (same rounding points: bf16 gate / up / h / down rows, bf16 low-rank intermediates and factors).  With few
 * tokens an expert sees one or two rows and the time is the bytes of the touched experts: each touched expert's three
 * matrices are streamed once, multiplied on the vector unit, in five launches on `stream` (four for up to four tokens).
 * xq_grouped_infer_supported() says whether a call fits: three banks of one format, block fp8 (fp32 scales), nvfp4
 * (GKN, e4m3 block scales, group 16) or nf4 (GKN, fp32 scales, group 64), that make an MLP, hidden and intermediate sizes multiples of 256, at most 1024 experts, 1..512 routed copies (n_tokens * topk), topk <= 16,
 * r in 1..64.  Other calls return XQ_ERR_ARG here: the caller takes xq_grouped_fwd for them.
 * workspace: xq_grouped_infer_workspace_bytes() bytes, 256-byte aligned. */
int xq_grouped_infer_supported(const xq_weight* gate, const xq_weight* up, const xq_weight* down, int64_t n_tokens,
                               int32_t topk, int r);
int64_t xq_grouped_infer_workspace_bytes(int64_t n_tokens, int32_t topk, int32_t num_experts, int64_t hidden,
                                         int64_t intermediate, int r);
int xq_grouped_fwd_infer(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                         const void* hidden, int64_t ld_hidden, int64_t n_tokens, const void* routing_w, int rw_dtype,
                         const int32_t* selected, int32_t topk, void* out, int64_t ld_out, void* workspace,
                         int64_t workspace_bytes, void* stream);

/* ---- the dense SwiGLU MLP in two calls ---------------------------------------
 * y = down(silu(gate(x)) * up(x)) over three QLoRA linears: the reference's Qwen3MLP.forward
 * (models/transformers/qwen3/modeling_qwen3.py:60-81) on QLoRALinear modules (qlora/modules/linear.py:369-385) with
 * fused_silu_and_mul between them (ops/fused_silu_and_mul.py:22-60), and its autograd backward.  Same arithmetic
 * and rounding points as three xq_linear_fwd calls around xq_silu_mul_fwd; what the separate calls repeat is
 * shared (one pass over x for both low-rank intermediates; block-fp8 gate / up as one launch that also writes the
 * SwiGLU output; the two input-gradient products as one launch; one pass over x for the two A gradients).
 *
 * Weights FLAT: gate, up [I, H], down [H, I] (H, I multiples of 64), any format.  LoRA factors in the dense module
 * layout, A[p] [r, in], B[p] [out, r] for p = 0 gate, 1 up, 2 down, fp32 or bf16, r in 0..64; bias[p] bf16 or NULL.
 * xq_mlp_saved names caller buffers the forward fills and the backward reads (r_pad = r rounded up to 16):
 * gate_up bf16 [M, 2 I] (gate | up), h bf16 [M, I], su_gate_up bf16 M * 2 * r_pad elements, su_down bf16
 * [M, r_pad]; the backward also reads x.  Factor gradients fp32, shaped like the factors, overwritten; dx may be
 * NULL.  workspace: xq_mlp_workspace_bytes(..., backward) bytes, 256-byte aligned. */
typedef struct xq_mlp_lora {
    const void* A[3];
    const void* B[3];
    const void* bias[3];
    int32_t dtype;      /* XQ_DT_* of all six factors */
    int32_t r;
    float scaling;
    int32_t reserved;
} xq_mlp_lora;

typedef struct xq_mlp_saved {
    void* gate_up;
    void* h;
    void* su_gate_up;
    void* su_down;
    /* How the forward ran gate and up, which fixes the layout of su_gate_up.  On entry to xq_mlp_fwd: < 0 lets the
     * process-wide default decide (xq_set_mlp_gate_up_fused), 0 asks for two launches, 1 for one launch with the SwiGLU in
     * its epilogue (block-fp8 gate and up only; otherwise two).  On return: 0 or 1, what was done.  xq_mlp_bwd reads it --
     * hand it the struct the forward filled (or the same value) -- and rejects anything else; the process-wide switch
     * plays no part in a backward. */
    int32_t gate_up_fused;
    int32_t reserved;
} xq_mlp_saved;

typedef struct xq_mlp_grads {
    float* dA[3];
    float* dB[3];
} xq_mlp_grads;

int64_t xq_mlp_workspace_bytes(int64_t M, int64_t hidden, int64_t intermediate, int r, int backward);
int xq_mlp_fwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
               const void* x, int64_t ldx, int64_t M, void* y, int64_t ldy, xq_mlp_saved* saved,
               void* workspace, int64_t workspace_bytes, void* stream);
int xq_mlp_bwd(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
               const void* x, int64_t ldx, const void* dy, int64_t lddy, int64_t M, const xq_mlp_saved* saved,
               void* dx, int64_t lddx, const xq_mlp_grads* grads, void* workspace, int64_t workspace_bytes,
               void* stream);

/* The same MLP forward when nothing is kept for a backward (inference, rollout: the reference's Qwen3MLP.forward under
 * torch.no_grad(), modeling_qwen3.py:60-81).  Each projection takes the kernel that suits the row count: up to 64 rows
 * the weight-streaming kernels (gate and up as one launch up to 16 rows), above that the tile kernels; the rounding
 * points are those of the separate module calls.  The intermediate gate|up and h live in the workspace
 * (xq_mlp_infer_workspace_bytes(...) bytes, 256-byte aligned). */
int64_t xq_mlp_infer_workspace_bytes(int64_t M, int64_t hidden, int64_t intermediate, int r);
int xq_mlp_fwd_infer(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_mlp_lora* lora,
                     const void* x, int64_t ldx, int64_t M, void* y, int64_t ldy, void* workspace,
                     int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* XQ_H */
