// Fused block-fp8 dequant-GEMM for dense weights, 256 x 256 x 64 tiles: both operand tiles come from global memory straight
// into LDS (global_load_lds, 16 bytes per lane: no trip through registers and no LDS store instruction for either
// operand), three LDS stages, the weight tile kept as its e4m3 BYTES in LDS and decoded after the fragment read, the
// products on v_mfma_f32_16x16x32_bf16.
//
//   C[rows, Nout] = A[rows, Kc] . Wop (+ su[rows, r] . Lr[Nout, r]^T) (+ bias)
//     CC  (dense forward): Wop[kc][n] = W[n][kc], W [Nout, Kc] bytes, fp32 scale per 128 x 128 block
//     !CC (dense dgrad):   Wop[kc][n] = W[kc][n], W [Kc, Nout] bytes; optionally over two matrices of one shape
//                          (G256Args::W2: K-steps from nk1 on read the second one)
//
// Same contract, arguments (G256Args) and tile order as gemm_256_kernel (xq_gemm_256.h), one block per tile.
//  * Why 16 x 16 x 32.  On operands that toggle (real data) the chip is power-limited, and this MFMA form moves half the
//    accumulator bytes per FLOP through the register file (a 16 x 16 fp32 tile per 16 K FLOP against a 32 x 32 tile per
//    32 K): an MFMA-only loop on N(0, 1) operands runs 1.9 PFLOP/s in this form against 1.65-1.7 in the 32 x 32 x 16 form
//    (both 2.46 on zeros).  A wave's 128 x 64 sub-tile is 8 x 4 MFMA tiles (128 accumulator registers); a K-step is two
//    k32 steps of 32 MFMAs.  Operand order (weight fragment, activation fragment) -> D[n][m]: lane l ends with output
//    row m = l % 16 and the 4 consecutive columns n = 4 (l / 16) ..
//  * Stages.  An activation stage is [256 rows][64 k] bf16, 16-byte chunk c of row r at chunk c ^ ((r >> 1) & 5); a weight
//    stage is [256 n][64 k] bytes (CC; chunk swizzle (n >> 2) & 2) or [64 k][256 n] bytes (!CC; chunk swizzle k & 7).  The
//    swizzles are made for the way the LDS serves a 16-byte read: it takes a wave's lanes {0-3, 12-15, 20-27}, {4-11, 16-19,
//    28-31} and the same two sets + 32 as four groups of 16, and the 16 lanes of a group must hit 16 different 16-byte
//    columns of the 64 banks (measured with a probe; with (r >> 1) & 7 and (n >> 2) & 3, which suit lanes 0-15 as a group,
//    these reads ran at half rate).  A
//    direct-to-LDS load writes lane l's 16 bytes at (wave-uniform base) + 16 l, so the swizzle is applied on the global
//    side: lane l fetches the chunk that belongs at its place.  48 KB per stage.
//  * Fragments.  In k32 step s lane group g = l / 16 takes k = 16 g + 8 s .. + 8 of the K-step's 64, so that a lane's
//    two steps are ONE 16-byte piece of a weight row (CC: one ds_read_b128 per weight tile and K-step; !CC: two
//    ds_read_b64_tr_b8, the transposing byte read, which hands lane i of a 16-lane group column i of an 8 x 16 byte
//    block); the activation fragments follow the same order: 16-byte chunk 2 g + s of row l % 16.
//  * Decode.  v_cvt_pk_f32_fp8, times the block scale (one scalar per wave and K-step, from a table in LDS),
//    v_cvt_pk_bf16_f32: bit for bit the bf16 the reference decoder produces (block_fp8_gkn_quantize.py:131-154).  A
//    weight value is decoded by the two waves that share its column block.
//  * Schedule.  A K-step is 16 chunks (step s, row tile i) of 4 MFMAs.  Activation fragments run through a ring of 4
//    register sets, each read three chunks ahead; the weight bytes of the NEXT K-step are read during chunks 8-11 and
//    its first step's operands decoded during chunks 12-15, the second step's during chunks 0-7 of its own iteration;
//    the six loads of K-step kt + 2 go out one per chunk.  Reads of the next stage start BEFORE the iteration's barrier,
//    which is possible because with three stages the loads of K-step j are made to land by the barrier of iteration
//    j - 2 (they are requested behind the barrier of iteration j - 3: one iteration in flight); the barrier sits at the
//    very end of an iteration and nothing waits behind it.
#pragma once

#include <type_traits>

#include "xq_gemm_256.h"

namespace xq {

struct GeoDtl {
    static constexpr int T = 256, NT = 512, BK = 64, STAGES = 3;
    static constexpr int A_STAGE_BYTES = T * BK * 2;    // 32 KB
    static constexpr int W_STAGE_BYTES = T * BK;        // 16 KB
    static constexpr int STAGE_BYTES = A_STAGE_BYTES + W_STAGE_BYTES;
    static constexpr int SCL_MAX = 256;                 // 128-k blocks of a contraction (Kc <= 32768)
    static constexpr size_t lds_bytes() { return (size_t)STAGES * STAGE_BYTES; }          // the operand stages
    static constexpr size_t lds_total() { return lds_bytes() + 2 * SCL_MAX * 4; }          // + the scales
};

#define XQ_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define XQ_GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// 4 e4m3 bytes (one dword) -> 4 bf16 (two dwords), each bf16(fl(e4m3 * sc))
__device__ __forceinline__ u32x2 dtl_decode4(uint32_t w, float sc) {
    const f32x2 x0 = e4m3x2_to_f32(w, false), x1 = e4m3x2_to_f32(w, true);
    return u32x2{pack_bf16x2(x0[0] * sc, x0[1] * sc), pack_bf16x2(x1[0] * sc, x1[1] * sc)};
}

// NW = 8: eight waves as 2 x 4, a wave 128 x 64 (two waves per SIMD).  NW = 4: four waves side by side, a wave 256 x 64
// with its 256 accumulator registers (one wave per SIMD): every weight value is then decoded by exactly one wave -- half
// the conversions per MFMA of the eight-wave form, whose column blocks are shared by two waves -- and an activation
// fragment feeds the same four MFMAs.
//
// GROUPED: the rows are in expert order and W is a bank of matrices of one shape (G256Args: offsets, tile_prefix,
// packed_stride, scale_stride, a_rows); a block finds the expert of its row tile, reads and writes that expert's rows only,
// and is gone if the launch holds fewer row tiles than its grid covers.  !CC is a bank's forward (optionally over two
// banks side by side: column tiles from ncols1 on take the second bank), CC its dgrad (optionally one sum over two banks:
// K-steps from nk1 on read the second one).
template <bool CC, int NW, bool GROUPED = false>
__global__ void __launch_bounds__(NW * 64, NW == 8 ? 2 : 1) gemm_dtl16_kernel(G256Args g) {
    using D = GeoDtl;
    constexpr int T = 256, TN = 4, NT = NW * 64;
    constexpr int RW = NW == 8 ? 128 : 256;          // rows of a wave's sub-tile
    constexpr int TM = RW / 16;                      // its row tiles: 8 or 16
    constexpr int NC = 2 * TM;                       // chunks of a K-step
    constexpr int AP = 32 / NW, WP = 16 / NW;        // direct loads per wave and K-step: activation rows, weight rows
    extern __shared__ __attribute__((aligned(16))) unsigned char dsm[];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = NW == 8 ? wave >> 2 : 0, wn = wave & 3;
    const int l16 = lane & 15, lg = lane >> 4;

    int pid_m, pid_n;
    {
        // (grouped: the grid covers an upper bound of the row tiles; the order is laid over the tiles there are, so that
        // the blocks with nothing to do are not all one XCD's)
        const int nb = (GROUPED ? g.tile_prefix[g.num_experts] : g.tiles_m) * g.tiles_n;
        const int b = blockIdx.x, per = nb >> 3;
        if (GROUPED && b >= nb) return;
        const int logical = (b < per * 8) ? (b & 7) * per + (b >> 3) : b;
        if constexpr (GROUPED) {
            pid_m = logical / g.tiles_n;      // all column tiles of a row tile side by side: an XCD stays on one expert's matrix
            pid_n = logical - pid_m * g.tiles_n;
        } else {
            constexpr int GM = 4;
            const int width = GM * g.tiles_n;
            const int grp = logical / width, first_m = grp * GM;
            const int gsz = min(g.tiles_m - first_m, GM);
            const int in = logical - grp * width;
            pid_m = first_m + in % gsz;
            pid_n = in / gsz;
        }
    }
    // the tile: expert, rows it may read and write, output columns (n0) and the same columns within their bank (n0w)
    int e = 0;
    int64_t row0 = (int64_t)pid_m * T, row_end = g.M;
    if constexpr (GROUPED) {
        // thread t looks at expert t (t + NT, ...): one memory round trip instead of a search's chain of dependent loads
        __shared__ int sh_tile[3];
        if (tid == 0) sh_tile[0] = -1;
        __syncthreads();
        for (int t = tid; t < g.num_experts; t += NT) {
            const int lo = g.tile_prefix[t], hi = g.tile_prefix[t + 1];
            if (lo <= pid_m && pid_m < hi) {
                sh_tile[0] = t;
                sh_tile[1] = g.offsets[t] + (pid_m - lo) * T;
                sh_tile[2] = g.offsets[t + 1];
            }
        }
        __syncthreads();
        e = __builtin_amdgcn_readfirstlane(sh_tile[0]);
        if (e < 0) return;                    // (cannot happen for a row tile below tile_prefix[num_experts])
        row0 = __builtin_amdgcn_readfirstlane(sh_tile[1]);
        row_end = __builtin_amdgcn_readfirstlane(sh_tile[2]);
    }
    const int n0 = pid_n * T;
    int n0w = n0, bank_width = g.Nout;
    const uint8_t* Wb = g.W + (int64_t)e * g.packed_stride;
    const float* Sb = (const float*)(g.scales + (int64_t)e * g.scale_stride);
    const float* Sb2 = g.W2 != nullptr ? (const float*)(g.scales2 + (int64_t)e * g.scale_stride) : nullptr;
    const bf16_t* su_b = g.su;
    const bf16_t* lr_b = g.lora_right;
    if constexpr (GROUPED && !CC) {
        if (g.W2 != nullptr) {
            bank_width = g.ncols1;
            if (n0 >= g.ncols1) {
                Wb = g.W2 + (int64_t)e * g.packed_stride; Sb = Sb2; su_b = g.su2; lr_b = g.lora_right2; n0w = n0 - g.ncols1;
            }
        }
    }
    const int nk = g.Kc / D::BK;
    const int scols = (g.wcols + 127) >> 7;
    // 16-row tiles of this wave's sub-tile that hold rows of the problem: the MFMAs of the others are skipped (their sums
    // would never be stored), so the last tile of an expert -- or of a dense matrix -- costs what its rows cost rounded up to
    // 16, not to 256: the two waves of a SIMD share its matrix pipe, and one of them leaving it alone hands it to the other
    const int mt = __builtin_amdgcn_readfirstlane((int)max((int64_t)0, min((int64_t)TM, (row_end - row0 - wm * RW + 15) >> 4)));

    // ---- direct-to-LDS sources (the stage layouts of gemm_dtl_kernel): a wave brings in the 8 AP activation rows from
    // wave * 8 AP on and the 16 WP weight rows (CC; !CC: 4 WP k rows) from wave * 16 WP (4 WP) on
    // A lane's source is (a base every lane shares, advanced from K-step to K-step in scalar registers) + (a 32-bit byte
    // offset of its own, fixed for the tile): the address costs no vector instruction per load.  (The host sends launches
    // whose activation matrix or weight matrix spans 4 GiB or more to gemm_256_kernel.)
    uint32_t a_off[AP];
#pragma unroll
    for (int p = 0; p < AP; ++p) {
        const int rt = (wave * AP + p) * 8 + (lane >> 3);
        int64_t r = row0 + rt;
        r = r < row_end ? r : row_end - 1;
        if constexpr (GROUPED) {
            if (g.a_rows) r = g.a_rows[r];
        }
        a_off[p] = (uint32_t)((r * g.lda + (((lane & 7) ^ ((rt >> 1) & 5)) << 3)) * 2);
    }
    uint32_t w_off[WP];
#pragma unroll
    for (int q = 0; q < WP; ++q) {
        if (CC) {
            const int rt = (wave * WP + q) * 16 + (lane >> 2);
            const int wr = min(n0w + rt, g.wrows - 1);
            w_off[q] = (uint32_t)((int64_t)wr * g.wcols + (((lane & 3) ^ ((rt >> 2) & 2)) << 4));
        } else {
            const int kr = (wave * WP + q) * 4 + (lane >> 4);
            const int wc = min(n0w + (((lane & 15) ^ (kr & 7)) << 4), g.wcols - 16);
            w_off[q] = (uint32_t)((int64_t)kr * g.wcols + wc);
        }
    }
    const int64_t w_kstep = CC ? D::BK : (int64_t)D::BK * g.wcols;
    // contraction over two matrices of one shape (dgrad of gate and up as one sum, G256Args::W2; dense: !CC, banks: CC):
    // K-steps from nk1 on read the second matrix (the same expert's), from its first K-step
    constexpr bool TWO_K = GROUPED ? CC : !CC;
    const int nk1 = (TWO_K && g.W2 != nullptr) ? g.nk1 : (1 << 30);
    const int64_t w2_delta = (TWO_K && g.W2 != nullptr) ? (g.W2 - g.W) - (int64_t)nk1 * w_kstep : 0;
    // (written out: the compiler's form of this load takes a 64-bit address per lane.  M0 -- the LDS base of the load -- is
    // written here and used nowhere else in the kernel: the compiler is not told, it has no use for M0 in this kernel.)
    const uint32_t dma_lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)dsm;
    auto issue_part = [&](int kt, int stage, int part) {
        const uint32_t a = dma_lds0 + stage * D::STAGE_BYTES + wave * (AP * 1024);
        const uint32_t w = dma_lds0 + stage * D::STAGE_BYTES + D::A_STAGE_BYTES + wave * (WP * 1024);
        if (part < AP) {
            const unsigned char* base = (const unsigned char*)(g.A + kt * D::BK);
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :: "s"(a + part * 1024), "v"(a_off[part]), "s"(base) : "memory");
        } else {
            const unsigned char* base = Wb + (kt * w_kstep + (kt >= nk1 ? w2_delta : 0));
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                         :: "s"(w + (part - AP) * 1024), "v"(w_off[part - AP]), "s"(base) : "memory");
        }
    };

    float* s_lds = (float*)(dsm + D::lds_bytes());
    {
        const int nkb = (nk + 1) >> 1;
        for (int i = tid; i < 2 * nkb; i += NT) {
            const int blk = i / nkb, kb = i - blk * nkb;
            const int nn = n0w + blk * 128;
            const bool second = 2 * kb >= nk1;                      // (nk1 is even: the matrices change on a scale-block boundary)
            const float* sp = second ? Sb2 : Sb;
            const int kb1 = second ? kb - (nk1 >> 1) : kb;
            float v;
            if (CC) v = sp[(min(nn, g.wrows - 1) >> 7) * scols + kb1];
            else v = sp[(int64_t)kb1 * scols + (min(nn, g.wcols - 1) >> 7)];
            s_lds[blk * D::SCL_MAX + kb] = v;
        }
        __syncthreads();
    }
    const float* sc_row = s_lds + (wn >> 1) * D::SCL_MAX;

    f32x4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- fragment reads.  They are written out as LDS instructions with the waits counted by hand: LDS operations of a
    // wave return in order, so "at most N newer reads outstanding" is an exact condition for a read to have landed, and
    // the ring below needs exactly that (left to the compiler, every wait in this loop came out as lgkmcnt(0), which
    // also waits for the read issued a few instructions earlier and exposes the whole LDS latency several times per
    // K-step).  No other LDS access is made inside the loop.
    const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)dsm;
    const int a_sw = (l16 >> 1) & 5;                                  // ((row >> 1) & 5) for every row tile
    // byte address (stage 0) of this lane's activation chunk of step s in row tile 0; + i * 2048 per row tile
    uint32_t a_addr[2];
#pragma unroll
    for (int s_ = 0; s_ < 2; ++s_) a_addr[s_] = lds0 + (wm * RW + l16) * 128 + ((((lg << 1) + s_) ^ a_sw) << 4);
    // weight bytes: CC one 16-byte read per tile (+ j * 1024); !CC two transposing 8-byte reads per tile (+ j * 16 columns
    // = the chunk index changes: one address per tile)
    uint32_t w_addr[CC ? 1 : 2 * TN];
    if constexpr (CC) {
        w_addr[0] = lds0 + D::A_STAGE_BYTES + (wn * 64 + l16) * 64 + ((lg ^ ((l16 >> 2) & 2)) << 4);
    } else {
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int kr = (lg << 4) + (h << 3) + (l16 >> 1);
                w_addr[2 * j + h] = lds0 + D::A_STAGE_BYTES + kr * 256 + (((wn * 4 + j) ^ (kr & 7)) << 4) + ((l16 & 1) << 3);
            }
    }
    constexpr int WREADS = CC ? 1 : 2;                                // LDS instructions per weight tile
    // (the reads take their offsets as immediates, so they are expanded from the chunk index at compile time)
#define XQ_DTL_READ_A(dst, so, c)                                                                                   \
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(a_addr[(c) / TM] + (so)), "n"(((c) % TM) * 2048))
#define XQ_DTL_READ_W(dst, so, j)                                                                                   \
    do {                                                                                                            \
        if constexpr (CC) {                                                                                         \
            asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(w_addr[0] + (so)), "n"((j) * 1024));     \
        } else {                                                                                                    \
            u32x2 lo_, hi_;                                                                                         \
            asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(lo_) : "v"(w_addr[CC ? 0 : 2 * (j)] + (so)));           \
            asm volatile("ds_read_b64_tr_b8 %0, %1" : "=v"(hi_) : "v"(w_addr[CC ? 0 : 2 * (j) + 1] + (so)));       \
            dst = u32x4{lo_[0], lo_[1], hi_[0], hi_[1]};                                                           \
        }                                                                                                           \
    } while (0)

    // ---- prologue: K-steps 0 and 1 requested and waited for (nk >= 3)
#pragma unroll
    for (int part = 0; part < AP + WP; ++part) issue_part(0, 0, part);
#pragma unroll
    for (int part = 0; part < AP + WP; ++part) issue_part(1, 1, part);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();

    bf16x8 fa[4];                 // ring: chunk c uses fa[c & 3]
    u32x4 fb0[TN], fb1[TN];       // decoded weight operands of step 0 / step 1 (8 bf16 each)
    u32x4 raw[TN];
    float sc = sc_row[0];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    XQ_DTL_READ_W(raw[0], 0u, 0); XQ_DTL_READ_W(raw[1], 0u, 1); XQ_DTL_READ_W(raw[2], 0u, 2); XQ_DTL_READ_W(raw[3], 0u, 3);
    XQ_DTL_READ_A(fa[0], 0u, 0); XQ_DTL_READ_A(fa[1], 0u, 1); XQ_DTL_READ_A(fa[2], 0u, 2);
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(raw[0]), "+v"(raw[1]), "+v"(raw[2]), "+v"(raw[3]), "+v"(fa[0]), "+v"(fa[1]), "+v"(fa[2]));
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const u32x2 d0 = dtl_decode4(raw[j][0], sc), d1 = dtl_decode4(raw[j][1], sc);
        fb0[j] = u32x4{d0[0], d0[1], d1[0], d1[1]};
    }

    // LDS instructions a chunk issues (after its MFMAs): its activation read, its weight reads, the scale read
    auto reads_in_chunk = [](int c, bool more) constexpr -> int {
        int n = (c + 3 < NC || more) ? 1 : 0;
        if (more && c >= TM && c < TM + 4) n += WREADS;
        if (more && c == 0) n += 1;
        return n;
    };

    int stage = 0;
    auto iteration = [&](int kt, auto MORE_, auto HAVE2_, auto SKIP_) {
        constexpr bool MORE = decltype(MORE_)::value, HAVE2 = decltype(HAVE2_)::value, SKIP = decltype(SKIP_)::value;
        const uint32_t so = (uint32_t)stage * D::STAGE_BYTES;
        const int nstage = stage == 2 ? 0 : stage + 1;
        const int pstage = stage == 0 ? 2 : stage - 1;        // stage of K-step kt + 2 (free since the last barrier)
        const uint32_t son = (uint32_t)nstage * D::STAGE_BYTES;
        float sc_next = sc;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const int i = c % TM;
            // the chunk's operands have landed when only the reads of the two chunks before this one are still out
            {
                const int n1 = c >= 1 ? reads_in_chunk(c - 1, MORE) : 0, n2 = c >= 2 ? reads_in_chunk(c - 2, MORE) : 0;
                const int n = n1 + n2;
                // (the registers named are the ones the following instructions consume: they may not be scheduled ahead of the wait)
                if (MORE && c >= TM + 4 && c < TM + 8) {
                    const int j = c - (TM + 4);
                    if (n == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                    else if (n == 3) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                    else if (n == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                    else if (n == 5) asm volatile("s_waitcnt lgkmcnt(5)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                    else if (n == 6) asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[c & 3]), "+v"(raw[j]));
                } else {
                    if (n == 1) asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else if (n == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else if (n == 3) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else if (n == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else if (n == 5) asm volatile("s_waitcnt lgkmcnt(5)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else if (n == 6) asm volatile("s_waitcnt lgkmcnt(6)" : "+v"(fa[c & 3]), "+v"(sc_next));
                    else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(fa[c & 3]), "+v"(sc_next));
                }
            }
            // the chunk's four MFMAs
            if (!SKIP || i < mt)
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                if constexpr (NW == 4) {
                    // (written out so that the accumulator stays where it is: left to itself the register allocator moves the
                    // 256 accumulator registers of this form between the two register files around every MFMA)
                    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(c < TM ? fb0[j] : fb1[j]), "v"(fa[c & 3]));
                } else {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, c < TM ? fb0[j] : fb1[j]), fa[c & 3], acc[i][j], 0, 0, 0);
                }
            }
            // the activation fragment three chunks on (the last three chunks fetch the next K-step's first three)
            if (c + 3 < NC) XQ_DTL_READ_A(fa[(c + 3) & 3], so, c + 3);
            else if (MORE) XQ_DTL_READ_A(fa[(c + 3) & 3], son, c + 3 - NC);
            // the next K-step's scale (chunk 0), weight bytes (their registers are free once the second step is decoded)
            if (MORE && c == 0) {
                const uint32_t sa = lds0 + (uint32_t)D::lds_bytes() + (uint32_t)(((wn >> 1) * D::SCL_MAX + ((kt + 1) >> 1)) * 4);
                asm volatile("ds_read_b32 %0, %1" : "=v"(sc_next) : "v"(sa));
            }
            if (MORE && c >= TM && c < TM + 4) XQ_DTL_READ_W(raw[c - TM], son, c - TM);
            // this K-step's second-step operands: 8 half tiles (4 values each) over the TM chunks of the first step
            if (c < TM && (TM == 8 || (c & 1) == 0)) {
                const int u = TM == 8 ? c : c >> 1, j = u >> 1, h = u & 1;
                const u32x2 d = dtl_decode4(raw[j][2 + h], sc);
                fb1[j][2 * h] = d[0];
                fb1[j][2 * h + 1] = d[1];
            }
            // the next K-step's first-step operands
            if (MORE && c >= TM + 4) {
                if constexpr (TM == 8) {
                    const int j = c - 12;
                    const u32x2 d0 = dtl_decode4(raw[j][0], sc_next), d1 = dtl_decode4(raw[j][1], sc_next);
                    fb0[j] = u32x4{d0[0], d0[1], d1[0], d1[1]};
                } else if (c < TM + 12) {
                    const int u = c - (TM + 4), j = u >> 1, h = u & 1;
                    const u32x2 d = dtl_decode4(raw[j][h], sc_next);
                    fb0[j][2 * h] = d[0];
                    fb0[j][2 * h + 1] = d[1];
                }
            }
            // the loads of K-step kt + 2, one per chunk
            if (HAVE2 && c < AP + WP) issue_part(kt + 2, pstage, c);
            __builtin_amdgcn_sched_barrier(0);
        }
        if (MORE) {
            // the loads of K-step kt + 2 have landed, and so have the fragment reads for the next iteration
            if (HAVE2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
            else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            __builtin_amdgcn_s_barrier();
        }
        sc = sc_next;
        stage = nstage;
    };
    {
        using Tt = std::integral_constant<bool, true>;
        using Ff = std::integral_constant<bool, false>;
        // (two copies of the loop: the one for whole tiles carries no test of the row tiles)
        auto run = [&](auto SKIP_) {
            int kt = 0;
            for (; kt + 2 < nk; ++kt) iteration(kt, Tt{}, Tt{}, SKIP_);
            iteration(kt, Tt{}, Ff{}, SKIP_);
            iteration(kt + 1, Ff{}, Ff{}, SKIP_);
        };
        if (mt == TM) run(Ff{});
        else run(Tt{});
    }
#undef XQ_DTL_READ_A
#undef XQ_DTL_READ_W

    // ---- low-rank side term: su[rows, rp] x lora_right[n, rp] as bf16 [row][64 k] tiles in the first two stages, k beyond
    // rp zero up to the next multiple of 32
    bf16_t* As = (bf16_t*)dsm;
    bf16_t* Bs = (bf16_t*)(dsm + D::STAGE_BYTES);
    __syncthreads();
    if (g.r_pad > 0) {
        const int rp = g.r_pad, steps = (rp + 31) >> 5, cpr = steps << 2, have = rp >> 3;
        const bf16_t* lr = lr_b + (int64_t)e * bank_width * rp;
        for (int idx = tid; idx < T * cpr; idx += NT) {
            const int r = idx / cpr, c = idx - r * cpr;
            int64_t row = row0 + r;
            row = row < row_end ? row : row_end - 1;
            int n = n0w + r;
            n = n < bank_width ? n : bank_width - 1;
            const u32x4 z = {0, 0, 0, 0};
            *(u32x4*)(As + swz(r, c)) = c < have ? *(const u32x4*)(su_b + row * g.ld_su + c * 8) : z;
            *(u32x4*)(Bs + swz(r, c)) = c < have ? *(const u32x4*)(lr + (int64_t)n * rp + c * 8) : z;
        }
        __syncthreads();
        for (int ks = 0; ks < steps; ++ks) {
            bf16x8 bw[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) bw[j] = *(const bf16x8*)(Bs + swz(wn * 64 + j * 16 + l16, ks * 4 + lg));
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const bf16x8 ax = *(const bf16x8*)(As + swz(wm * RW + i * 16 + l16, ks * 4 + lg));
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if constexpr (NW == 4) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(bw[j]), "v"(ax));
                    else acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bw[j], ax, acc[i][j], 0, 0, 0);
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }

    // ---- the finished tile.  Lane l holds, per (i, j) tile, row 16 i + l % 16 and the 4 columns 16 j + 4 (l / 16) ..: 8 bytes
    // of bf16.  Each wave passes its RW x 64 sub-tile through a private LDS area ([row][64] bf16, chunk swizzle) and writes
    // whole 128-byte row pieces, 8 rows per instruction.
    if constexpr (NW == 4) asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");     // the last MFMA results, written outside the compiler's hazard tracking
    bf16_t* stg = (bf16_t*)dsm + wave * (RW * 64);
    int lv = lane;
    asm volatile("" : "+v"(lv));
    const int s16 = lv & 15, sg = lv >> 4;
    const bool wide = g.wide_rows != 0;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        float b4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (g.bias) {
            const u32x2 b = *(const u32x2*)(g.bias + min(n0 + wn * 64 + j * 16 + 4 * sg, g.Nout - 4));
            b4[0] = __uint_as_float(b[0] << 16); b4[1] = __uint_as_float(b[0] & 0xffff0000u);
            b4[2] = __uint_as_float(b[1] << 16); b4[3] = __uint_as_float(b[1] & 0xffff0000u);
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const u32x2 v = {pack_bf16x2(acc[i][j][0] + b4[0], acc[i][j][1] + b4[1]), pack_bf16x2(acc[i][j][2] + b4[2], acc[i][j][3] + b4[3])};
            if (wide) {
                *(u32x2*)(stg + swz(i * 16 + s16, 2 * j + (sg >> 1)) + 4 * (sg & 1)) = v;
            } else {
                const int64_t row = row0 + wm * RW + i * 16 + s16;
                const int n = n0 + wn * 64 + j * 16 + 4 * sg;
                if (row < row_end && n < g.Nout) *(u32x2*)(g.C + row * g.ldc + n) = v;
            }
        }
    }
    if (wide) {
#pragma unroll
        for (int t = 0; t < RW / 8; ++t) {
            const int rl = t * 8 + (lv >> 3), ch = lv & 7;
            const u32x4 v = *(const u32x4*)(stg + swz(rl, ch));
            const int64_t row = row0 + wm * RW + rl;
            const int n = n0 + wn * 64 + ch * 8;
            if (row < row_end && n < g.Nout) *(u32x4*)(g.C + row * g.ldc + n) = v;
        }
    }
}

}  // namespace xq
