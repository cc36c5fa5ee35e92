// Large-M fused dequant-GEMM for block-fp8 weights: 256x256x64 tiles, 8 waves
// (2 along M x 4 along N, two per SIMD so one wave's LDS/VALU work hides under the
// other's MFMAs), each wave a 128x64 sub-tile of 4x2 v_mfma_f32_32x32x16_bf16
// whose 128 fp32 accumulators live in AGPRs.
//
//   C[M, Nout] = A[M, Kc] . Wop (+ su[M, r] . Lr[Nout, r]^T) (+ bias)
//
// W is e4m3 [wrows, wcols] with fp32 scales per 128x128 block.
//   CONTRACT_COLS (forward):  Wop[kc][n] = W[n][kc]; the decoded tile is stored
//     in LDS as [n][kc] (kc contiguous, XOR-swizzled 16-byte chunks) and read
//     with ds_read_b128 in MFMA operand order.
//   !CONTRACT_COLS (dgrad):   Wop[kc][n] = W[kc][n]; the decoded tile is stored
//     as it lies in memory, [kc][n], and the operand fragments are read with the
//     transposing LDS load ds_read_b64_tr_b16 -- no transposed copy of the
//     weight exists anywhere.
// Every fp8 byte is decoded exactly once per tile, in registers, to the bf16
// value the reference decoder produces (bf16(fl(float(e4m3) * scale))).
// LDS is double buffered; the next tile's global loads are issued first, its
// LDS stores and fp8 decode are spread between the four k16 MFMA groups of the
// current tile, and operand fragments are fetched one k16 step ahead.  Operands are swapped in the MFMA (D = W_frag x
// A_frag) so that each lane ends up with 4 consecutive output columns and the
// epilogue writes 8-byte packed bf16.
#pragma once

#include "xq_common.h"
#include "xq_gemm_tile.h"

namespace xq {

constexpr int F8_BM = 256, F8_BN = 256, F8_BK = 64;
constexpr int F8_A_STAGE = F8_BM * F8_BK;             // bf16 elements (32 KB)
constexpr int F8_NN_PITCH = F8_BN + 32;               // [kc][n] rows of 576 B
constexpr int F8_B_STAGE_NT = F8_BN * F8_BK;          // 32 KB
constexpr int F8_B_STAGE_NN = F8_BK * F8_NN_PITCH;    // 36 KB

// element offset of 16-byte chunk `c` (0..7) of row `r` in a [rows][64] bf16 tile.
// gfx950 LDS has 64 banks (256 B/clk) and serves a ds_read_b128 sixteen lanes at a
// time: 16 consecutive rows (128 B each, so even/odd rows sit in different bank
// halves) must land on 8 distinct chunk slots per parity -> XOR with (r >> 1) & 7.
__device__ __forceinline__ int swz(int r, int c) { return r * 64 + ((c ^ ((r >> 1) & 7)) << 3); }

struct Fp8Args {
    const bf16_t* A;
    int64_t lda;
    bf16_t* C;
    int64_t ldc;
    const uint8_t* W;
    const float* scales;
    int32_t wrows, wcols;
    int32_t Kc, Nout;
    int64_t M;
    const bf16_t* su;          // [M, r_pad] or NULL
    const bf16_t* lora_right;  // [Nout, r_pad] or NULL
    int32_t r_pad;
    const bf16_t* bias;
    int32_t tiles_m, tiles_n;
};

template <bool CC>
__global__ void __launch_bounds__(512, 2) gemm_fp8_256_kernel(Fp8Args g) {
    extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
    constexpr int B_STAGE = CC ? F8_B_STAGE_NT : F8_B_STAGE_NN;
    bf16_t* As = smem;                    // 2 stages
    bf16_t* Bs = smem + 2 * F8_A_STAGE;   // 2 stages

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 2, wn = wave & 3;   // wave tile: rows wm*128.., cols wn*64..

    // ---- XCD-aware tile mapping: consecutive workgroup ids land on different
    // XCDs, so give each XCD a contiguous range of logical tiles, and walk the
    // logical tiles in groups of 4 row-tiles so concurrent tiles share operands in L2.
    int pid_m, pid_n;
    {
        const int nb = g.tiles_m * g.tiles_n;
        int b = blockIdx.x;
        const int per = nb >> 3;
        int logical = (b < per * 8) ? (b & 7) * per + (b >> 3) : b;
        constexpr int GM = 4;
        const int width = GM * g.tiles_n;
        const int grp = logical / width, first_m = grp * GM;
        const int gsz = min(g.tiles_m - first_m, GM);
        const int in = logical - grp * width;
        pid_m = first_m + in % gsz;
        pid_n = in / gsz;
    }
    const int64_t row0 = (int64_t)pid_m * F8_BM;
    const int n0 = pid_n * F8_BN;
    const int scols = (g.wcols + 127) >> 7;

    // ---- per-thread global addresses (fixed across K-steps except for the k offset)
    const bf16_t* a_src[4];
    int a_dst[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int u = tid + p * 512;
        int64_t r = row0 + (u >> 3);
        r = r < g.M ? r : g.M - 1;
        a_src[p] = g.A + r * g.lda + (u & 7) * 8;
        a_dst[p] = swz(u >> 3, u & 7);
    }
    const uint8_t* w_src[2];
    const float* s_src[2];
    int w_dst[2];
    int64_t w_kstep, s_kstep_num;  // advance per K-step
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int u = tid + p * 512;
        int wr, wc;
        if (CC) { wr = min(n0 + (u >> 2), g.wrows - 1); wc = (u & 3) * 16; }
        else { wr = u >> 4; wc = min(n0 + (u & 15) * 16, g.wcols - 16); }
        w_src[p] = g.W + (int64_t)wr * g.wcols + wc;
        s_src[p] = g.scales + (CC ? (wr >> 7) * scols : (wc >> 7));
        w_dst[p] = CC ? (u >> 2) * 64 : (u >> 4) * F8_NN_PITCH + (u & 15) * 16;
    }
    w_kstep = CC ? F8_BK : (int64_t)F8_BK * g.wcols;
    (void)s_kstep_num;

    u32x4 areg[4];
    u32x4 wreg[2];
    float wscale[2];

    auto load_a = [&](int kt) {
        const int k0 = kt * F8_BK;
#pragma unroll
        for (int p = 0; p < 4; ++p) areg[p] = *(const u32x4*)(a_src[p] + k0);
    };
    auto load_w = [&](int kt) {
        const int k0 = kt * F8_BK;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            wreg[p] = *(const u32x4*)(w_src[p] + kt * w_kstep);
            wscale[p] = CC ? s_src[p][k0 >> 7] : s_src[p][(k0 >> 7) * scols];
        }
    };
    auto store_a = [&](bf16_t* a) {
#pragma unroll
        for (int p = 0; p < 4; ++p) *(u32x4*)(a + a_dst[p]) = areg[p];
    };
    auto store_w = [&](bf16_t* b, int p) {
        const float s = wscale[p];
        u32x4 lo, hi;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x2 x0 = e4m3x2_to_f32(wreg[p][i], false), x1 = e4m3x2_to_f32(wreg[p][i], true);
            uint32_t v0 = pack_bf16x2(x0[0] * s, x0[1] * s), v1 = pack_bf16x2(x1[0] * s, x1[1] * s);
            if (i < 2) { lo[2 * i] = v0; lo[2 * i + 1] = v1; }
            else { hi[2 * (i - 2)] = v0; hi[2 * (i - 2) + 1] = v1; }
        }
        if (CC) {
            const int u = tid + p * 512, r = u >> 2, c = (u & 3) * 2;
            *(u32x4*)(b + swz(r, c)) = lo;
            *(u32x4*)(b + swz(r, c + 1)) = hi;
        } else {
            *(u32x4*)(b + w_dst[p]) = lo;
            *(u32x4*)(b + w_dst[p] + 8) = hi;
        }
    };

    f32x16 acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;

    const int fr = lane & 31, fh = lane >> 5;
    auto load_frags = [&](const bf16_t* a, const bf16_t* b, int ks, bool b_is_nt, bf16x8* af, bf16x8* bfr) {
#pragma unroll
        for (int i = 0; i < 4; ++i) af[i] = *(const bf16x8*)(a + swz(wm * 128 + i * 32 + fr, ks * 2 + fh));
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (CC || b_is_nt) bfr[j] = *(const bf16x8*)(b + swz(wn * 64 + j * 32 + fr, ks * 2 + fh));
            else bfr[j] = lds_tr_frag(b, F8_NN_PITCH, ks * 16, wn * 64 + j * 32, lane);
        }
    };
    auto mma = [&](const bf16x8* af, const bf16x8* bfr) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[j], af[i], acc[i][j], 0, 0, 0);
    };

    // Pipeline: at the top of iteration kt the registers hold tile kt+1 (loaded one
    // whole iteration earlier, so the global latency is covered by a full tile of
    // MFMAs) and the operand fragments of k16-step 0 of tile kt.  Tile kt+1 is
    // stored/decoded into the other LDS stage and the loads of tile kt+2 are issued
    // while steps 0..2 are multiplied; the single barrier of the iteration sits before
    // the last step, whose MFMAs then cover both the barrier skew and the fetch of the
    // next tile's first fragments.  (Every read of a stage completes before the barrier
    // that precedes the next stores into it.)
    const int nk = g.Kc / F8_BK;
    bf16x8 af0[4], bf0[2], af1[4], bf1[2];
    auto iteration = [&](int kt, bool have_next, bool have_next2) {
        const bf16_t* a = As + (kt & 1) * F8_A_STAGE;
        const bf16_t* b = Bs + (kt & 1) * B_STAGE;
        bf16_t* an = As + ((kt + 1) & 1) * F8_A_STAGE;
        bf16_t* bn = Bs + ((kt + 1) & 1) * B_STAGE;
        // region 1: MFMAs of step 0 over the step-1 fragment reads, the A-tile stores and the next A loads
        mma(af0, bf0);
        load_frags(a, b, 1, false, af1, bf1);
        if (have_next) store_a(an);
        if (have_next2) load_a(kt + 2);
        // interleave: one LDS read behind each of the first six MFMAs, then the stores and global loads
        for (int q = 0; q < 6; ++q) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
        for (int q = 0; q < 2; ++q) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
        // region 2: MFMAs of step 1 over the weight decode + stores, the next weight loads, step-2 fragment reads
        mma(af1, bf1);
        if (have_next) { store_w(bn, 0); store_w(bn, 1); }
        if (have_next2) load_w(kt + 2);
        load_frags(a, b, 2, false, af0, bf0);
        __builtin_amdgcn_sched_barrier(0);
        // region 3: MFMAs of step 2 over the step-3 fragment reads
        mma(af0, bf0);
        load_frags(a, b, 3, false, af1, bf1);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
        // region 4: MFMAs of step 3 over the next tile's first fragment reads, which must have
        // landed before the next iteration starts multiplying
        if (have_next) load_frags(an, bn, 0, false, af0, bf0);
        mma(af1, bf1);
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    };
    load_a(0);
    load_w(0);
    store_a(As);
    store_w(Bs, 0);
    store_w(Bs, 1);
    if (nk > 1) { load_a(1); load_w(1); }
    __syncthreads();
    load_frags(As, Bs, 0, false, af0, bf0);
    int kt = 0;
    for (; kt + 2 < nk; ++kt) iteration(kt, true, true);
    if (kt + 1 < nk) { iteration(kt, true, false); ++kt; }
    iteration(kt, false, false);

    // ---- low-rank side term: su[rows, rp] x lora_right[n, rp], both [row][k] tiles in stage 0
    if (g.r_pad > 0) {
        const int rp = g.r_pad, cpr = rp >> 3;  // 16-byte chunks per row
        for (int idx = tid; idx < 256 * cpr; idx += 512) {
            const int r = idx / cpr, c = idx - r * cpr;
            int64_t row = row0 + r;
            row = row < g.M ? row : g.M - 1;
            *(u32x4*)(As + swz(r, c)) = *(const u32x4*)(g.su + row * rp + c * 8);
            int n = n0 + r;
            n = n < g.Nout ? n : g.Nout - 1;
            *(u32x4*)(Bs + swz(r, c)) = *(const u32x4*)(g.lora_right + (int64_t)n * rp + c * 8);
        }
        __syncthreads();
        for (int ks = 0; ks < (rp >> 4); ++ks) {
            bf16x8 af[4], bfr[2];
            load_frags(As, Bs, ks, true, af, bfr);
            mma(af, bfr);
        }
    }

    // ---- epilogue: lane holds, per (i, j) tile, row m = fr and 4 x 4 consecutive columns
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = row0 + wm * 128 + i * 32 + fr;
        if (row >= g.M) continue;
        bf16_t* crow = g.C + row * g.ldc;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int n = n0 + wn * 64 + j * 32 + 8 * q4 + 4 * fh;
                if (n >= g.Nout) continue;  // Nout % 16 == 0: groups of 4 are all in or all out
                float v0 = acc[i][j][4 * q4], v1 = acc[i][j][4 * q4 + 1], v2 = acc[i][j][4 * q4 + 2], v3 = acc[i][j][4 * q4 + 3];
                if (g.bias) {
                    v0 += bf16_to_f32(g.bias[n]); v1 += bf16_to_f32(g.bias[n + 1]);
                    v2 += bf16_to_f32(g.bias[n + 2]); v3 += bf16_to_f32(g.bias[n + 3]);
                }
                *(u32x2*)(crow + n) = u32x2{pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
            }
        }
    }
}

}  // namespace xq
