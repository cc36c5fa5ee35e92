// Skinny-M forward for M <= 16 in ONE launch (the decode regime: a handful of tokens against a large packed weight).
//
//   y[M, N] = x[M, K] . deq(W)^T + bias + s * (x . A^T) . B^T          (W FLAT [N, K])
//
// A block owns 16 G weight rows over the WHOLE of K: its 8 waves split K eight ways, sum their 16 x 16 tiles through LDS
// and write the outputs themselves -- no fp32 partial tiles in memory, no second launch.  All of a wave's loads are
// unconditional (clamped, masked): the x slice first (it reaches LDS while the weight bytes stream), then the weights
// as a stream with a few loads per lane in flight; every weight byte is read once, decoded in registers to the exact
// bf16 value of the reference decoder
// and fed to v_mfma_f32_16x16x32_bf16 against x fragments (lane (row, quarter) holds 16 or 32 consecutive codes of its
// row; the K order inside an MFMA is whatever the loads deliver, the x fragments follow the same order).
//
// The low-rank intermediate su = x . A^T [M, r] is needed whole by every block but costs r x K factor bytes to form, more
// than a block's share of the weight.  It is formed once per launch: in each of the first K / 512 blocks the four waves
// that are last in the load queue contract 512 elements of K before they turn to their weight rows, and publish the
// 256 sums to a slot in device memory; wave 0 of every block, which is the first to finish its part of the weight
// stream, collects the parts while the other waves are still streaming.  Nothing on that path waits for an atomic's
// return value or for an ordering between stores:
//  * the slot holds a launch count `gen`, which wave 0 of every block reads (behind its weight loads);
//  * a published entry is the 8-byte pair (sum, gen + 1), stored whole; a collector takes an entry when its tag is
//    gen + 1, so what earlier launches left in the slot never passes for this launch's sums and nothing is cleared;
//  * `gen` moves on once per launch, after every block has read it: each block adds one to `started` when its own read
//    has returned (no return value asked for), and the last block of the grid, which reads `started` along with the
//    parts, stores gen + 1 and started = 0 when it finds the whole grid there (it looks again if not).  Both words
//    exist in 32 copies on different memory lines (block b reads and counts in copy b % 32; the last block sums and
//    rewrites them all): hundreds of accesses to one location that bypass the caches would take microseconds.
// Slot accesses are device-scope atomics (they bypass the per-XCD L2s) unless said otherwise where they are made.
// Blocks that publish never wait, and they are the first the dispatcher places, so the collectors' wait ends; a limit
// bounds every wait all the same and turns the block's outputs into NaN.  A last block that gives up stores a mark in
// place of the launch count; every block that reads the mark -- late blocks of that launch, all blocks of later launches
// on the slot -- publishes nothing and writes NaN until the host clears the slots (reset_skinny_rows_slots): a failed
// launch never lets stale sums through.  Sums run in fixed orders (waves ascending, parts ascending): results are
// identical from call to call.
//
// Measured on an MI355X, launches back to back (block_fp8, r = 16, M = 1): 4096->12288 (48 MiB) 11.4 us against 15.6 us
// for the two-launch organisation (10.0 us without a low-rank term), 4096->4096 7.4 against 8.8, 4096->24576 (96 MiB)
// 18.4 against 22.1.
#include <stdlib.h>

#include <atomic>
#include <mutex>

#include "xq_common.h"
#include "xq_lora.h"
#include "xq_skinny.h"
#include <type_traits>

namespace xq {

constexpr int kSuPartK = 512;                   // K elements per su part
constexpr int kSuMaxParts = 32;                 // K <= 16384 with a low-rank term
constexpr int kSlotCtl = kSuMaxParts * 256 * 2; // word index of the control words
constexpr int kCtlCopies = 32;                  // `gen` and `started` exist 32 times, 128 bytes apart: block b uses copy b % 32,
constexpr int kCtlStride = 32;                  // so that a launch's 256 blocks do not queue on one memory location
constexpr int kSlotWords = kSlotCtl + 2 * kCtlCopies * kCtlStride;   // [parts][256] pairs (sum bits, tag), gen copies, started copies
constexpr int kSlots = 256;
constexpr int kRowsSpinLimit = 1 << 20;
constexpr uint32_t kGenPoison = 0xFFFFFFFFu;   // launch count of a slot in which a wait has given up: see the closer below
#ifndef XQ_ROWS_LOADS_IN_FLIGHT
#define XQ_ROWS_LOADS_IN_FLIGHT 6
#endif
constexpr int kRowsLoadsInFlight = XQ_ROWS_LOADS_IN_FLIGHT;   // 16-byte weight loads per lane kept in flight

struct SkinnyRowsArgs {
    const bf16_t* x;
    int64_t ldx;
    int32_t M, N, K;
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int32_t gshift, scale_dtype;   // int4: log2(group)
    const float* lora_A;           // [r, K] fp32
    const float* lora_B;           // [N, r] fp32
    int32_t r;
    float su_scale;
    const bf16_t* bias;
    bf16_t* y;
    int64_t ldy;
    int32_t xpitch, slab;          // bytes: LDS row pitch of a wave's x slice, bytes of a wave's LDS area
    int32_t nsu;                   // su parts (K / 512), 0 without a low-rank term
    uint32_t* slot;                // [nsu][256] published (sum, tag) pairs, then the copies of gen and of started
    int32_t spin_limit;
    uint32_t* fail;                // the device's count of blocks whose wait gave up (they wrote NaN): read by skinny_rows_status
};

// FMT: weight format; G: 16-row groups in flight per block; NJ: most load steps per wave (a step is one 16-byte load
// per lane: 64 elements of K per row for fp8, 128 for the 4-bit formats); MR: bound on M (x rows kept in registers on
// their way to LDS); R: rounds -- a block walks R sets of G row groups, each step's registers refilled for the next
// round as soon as the step has been multiplied, so the weight stream never stops (N % (16 G R) == 0 when R > 1)
// (`bx` of `nb`: the block's place among the blocks of its forward -- the grid of a launch holds one forward or several)
// GU (two rounds only): the weight is gate | up stacked, [2 I, K]; round 0 walks the block's gate rows and round 1 the up rows
// of the same columns, I rows further on, and the finish writes h[m][n] = bf16(bf16(silu(gate)) * up) from the two rounded
// outputs (ops/fused_silu_and_mul.py:22-60) to y [M, I] instead of the two outputs themselves.
template <int FMT, int G, int NJ, int MR, int R, bool PRE = false, bool GU = false>
__device__ __forceinline__ void skinny_rows_body(const SkinnyRowsArgs& g, const int bx, const int nb) {
    static_assert(!GU || R == 2, "the SwiGLU finish pairs the two rounds of a block");
    constexpr bool F8 = FMT == XQ_FMT_FP8;
    constexpr int EPS = F8 ? 64 : 128;                 // K elements of a row per load step
    constexpr int MPS = EPS / 32;                      // MFMAs per step and row group
    constexpr int EB = F8 ? 1 : 2;                     // elements per byte
    constexpr int XC = (NJ * EPS + 511) / 512;         // 1 KB pieces of an x row slice
    constexpr int NSC = FMT == XQ_FMT_NVFP4 ? 2 : 1;   // scale registers per load
    // every argument in scalar registers after one round trip (lazily placed argument loads cost a round trip each)
    if constexpr (!PRE)
        asm volatile("" ::"s"(g.x), "s"(g.ldx), "s"(g.M), "s"(g.N), "s"(g.K), "s"(g.packed), "s"(g.scales), "s"(g.global_scale),
                     "s"(g.gshift), "s"(g.scale_dtype), "s"(g.lora_A), "s"(g.lora_B), "s"(g.r), "s"(g.su_scale), "s"(g.bias), "s"(g.y),
                     "s"(g.ldy), "s"(g.xpitch), "s"(g.slab), "s"(g.nsu), "s"(g.slot), "s"(g.spin_limit));
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int rn = lane & 15, kq = lane >> 4;
    const int ks = g.K >> 3;                    // K elements per wave
    const int k0 = wave * ks;
    const int nj = ks / EPS;                    // load steps of this launch, 1 .. NJ
    const int n0 = bx * (16 * G * (GU ? 1 : R));
    const int rstride = GU ? g.N >> 1 : 16 * G;        // rows from a round's rows to the next round's
    const int nlim = GU ? g.N >> 1 : g.N;              // end of the rows that round 0 may walk
    const int XP = g.xpitch;
    unsigned char* slab = smem + wave * g.slab;
    float* su_tot = (float*)(smem + 8 * g.slab);           // [16 m][16 j], then a flag
    float* b_tile = su_tot + 272;                           // [96 rows][20]: the block's rows of B, 16 bytes apart in banks
    float* su_red = b_tile + 96 * 20;                       // [4 waves][256]: the tiles of an su part
    int* su_flag = (int*)(su_red + 4 * 256);                // [0 .. 3]: wave 4 + w has written its tile; [4]: wave 4 is done with `gen`
    const bool lora = g.nsu > 0;
    const bool su_block = bx < g.nsu;          // nsu <= nb (checked on the host)
    // LDS traffic of the block is ordered by this barrier; __syncthreads() would also wait for every load in flight
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };

    if (su_block) {
        // nothing is in flight yet: this barrier costs nothing, and LDS does not start out zero
        if (tid < 8) su_flag[tid] = 0;
        lds_barrier();
    }

    // ---- the slot's launch count.  A block that forms an su part has its publishing wave ask for it first of all (the part
    // carries it as its tag); everywhere wave 0 asks for it, past the caches, behind its weights (needed when it collects;
    // loads return in order and this one is slow, so it must not sit in front of them).
    uint32_t gen = 0;
    uint32_t* ctl = g.slot + kSlotCtl + (bx % kCtlCopies) * kCtlStride;      // this block's copy of gen; started: + kCtlCopies * kCtlStride

    // the operand tie keeps the compiler from moving the add ahead of the point where `gen` is in its register
    auto count_block = [&]() {
        uint32_t one = 1u;
        asm volatile("" : "+v"(one) : "v"(gen));
        __hip_atomic_fetch_add(ctl + kCtlCopies * kCtlStride, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };

    // ---- a block that forms an su part does so with its waves 4 .. 7: behind the others in the load queue, they would
    // otherwise sit waiting to issue their weight loads.  Wave 4 + w contracts elements 128 w .. of the part in four
    // MFMAs, lane (rank rn, quarter kq) holding 8 consecutive elements per MFMA; factor rows and x fragments are its
    // first loads.
    const bool su_wave = su_block && wave >= 4;
    u32x4 fa0[4], fa1[4];
    bf16x8 fx[4];
    if (su_wave) {
        __builtin_amdgcn_s_setprio(3);          // ahead of the other waves' loads: everyone's finish waits for these sums
        // the publisher tags the sums with it.  This read may come from the XCD's L2: no line of the slot can be there from
        // before the launch (caches are invalidated between kernels, or results could not pass from one kernel to the
        // next), and within a launch the word changes only after every block has read it.  A read past the caches takes
        // microseconds here, and every block's finish waits for the sums.  (Were the value stale after all, the tag
        // would not be the one the collectors look for: they would give up and write NaN, never take old sums.)
        if (wave == 4) gen = __hip_atomic_load(ctl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        const int kb = bx * kSuPartK + (wave - 4) * 128 + kq * 8;
        const float* ap = g.lora_A + (int64_t)(rn < g.r ? rn : 0) * g.K + kb;
        const bf16_t* xp = g.x + (int64_t)(rn < g.M ? rn : g.M - 1) * g.ldx + kb;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            fa0[u] = *(const u32x4*)(ap + u * 32);
            fa1[u] = *(const u32x4*)(ap + u * 32 + 4);
            fx[u] = *(const bf16x8*)(xp + u * 32);
        }
        __builtin_amdgcn_s_setprio(0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- x slice [M][ks] of this wave: a load instruction covers 1 KB of one row; rows past M and pieces past the slice
    // are clamped (loaded, never stored)
    u32x4 xr[MR][XC];
    const int ppr = ks >> 3;                    // 16-byte pieces per row of the slice
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < XC; ++c) {
            const int piece = c * 64 + lane < ppr ? c * 64 + lane : ppr - 1;
            xr[i][c] = *(const u32x4*)(g.x + (int64_t)(i < g.M ? i : g.M - 1) * g.ldx + k0 + piece * 8);
        }
    __builtin_amdgcn_sched_barrier(0);


    // ---- su part, before these waves' weight loads are requested: D[j][m] of each wave, the four tiles summed through LDS in
    // wave order by wave 4, published.  The waves meet through flags in LDS, not a barrier.
    if (su_wave) {
        f32x4 su = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            u32x4 t = {pack_bf16x2(__uint_as_float(fa0[u][0]), __uint_as_float(fa0[u][1])), pack_bf16x2(__uint_as_float(fa0[u][2]), __uint_as_float(fa0[u][3])),
                       pack_bf16x2(__uint_as_float(fa1[u][0]), __uint_as_float(fa1[u][1])), pack_bf16x2(__uint_as_float(fa1[u][2]), __uint_as_float(fa1[u][3]))};
            if (rn >= g.r) t = u32x4{0, 0, 0, 0};
            su = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, t), fx[u], su, 0, 0, 0);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) su_red[(wave - 4) * 256 + q * 64 + lane] = su[q];
        // the flag goes behind the tile: LDS operations of one wave execute in order.  (A release / acquire pair of the
        // language would also wait for every global load these waves have in flight -- their x slices.)
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if (lane == 0) __hip_atomic_store(su_flag + wave - 4, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        if (wave == 4) {
            int spins = 0;
            bool all;
            do {
                all = lane >= 4 || __hip_atomic_load(su_flag + (lane & 3), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0;
                all = __all(all);
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                if (!all) {
                    __builtin_amdgcn_s_sleep(2);
                    ++spins;
                }
            } while (!all && spins < g.spin_limit);
            // (a wait that hit the limit, or a slot that is marked failed, leaves the part unpublished: the collectors then
            // hit their limit, or see the mark, and write NaN)
            if (all && gen != kGenPoison) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float s = 0.0f;
#pragma unroll
                    for (int ww = 0; ww < 4; ++ww) s += su_red[ww * 256 + q * 64 + lane];
                    __hip_atomic_store((uint64_t*)g.slot + bx * 256 + q * 64 + lane, ((uint64_t)(gen + 1) << 32) | __float_as_uint(s),
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
            // wave 0 counts the block in once it has read `gen` itself, and not before this wave has
            if (lane == 0) __hip_atomic_store(su_flag + 4, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __builtin_amdgcn_sched_barrier(0);

    // ---- the block's weight rows, this wave's K range: step j gives lane (row rn, quarter kq) the 16 bytes at element
    // EPS j + (EPS / 4) kq of its row's slice.  The R NJ steps of a wave form one stream through a ring of DJ step
    // registers: DJ steps are requested up front, and each step's registers are refilled with the step DJ further on as
    // soon as it has been multiplied.  About 6 KB per wave in flight (48 KB per CU; 4 to 12 KB measure alike, 24 KB 10 % slower) keeps the memory pipe full (a CU takes loads only
    // as fast as memory returns them: more would queue in front of the other waves') and lets all eight waves advance
    // together, so that at the end only the last steps remain to be decoded.
    constexpr int T = R * NJ;                                   // steps of the stream (those past nj of a round are idle)
    constexpr int DJ = T < (kRowsLoadsInFlight + G - 1) / G ? T : (kRowsLoadsInFlight + G - 1) / G;
    u32x4 w[DJ][G];
    uint32_t sc[DJ][G][NSC];
    // int4 with one bf16 scale per 128 elements (a step): a lane's scales of four consecutive steps are 8 contiguous bytes,
    // and one load per four steps fetches them.  A 2-byte load per step and row group is a vector memory instruction that
    // touches 16 cache lines like the step's weight load itself -- as many instructions again as the weights take, and
    // the kernel runs at the pace of its memory instructions.  (Needs whole groups of four steps per wave, all in use.)
    constexpr bool I4 = FMT == XQ_FMT_INT4;
    const bool vs = I4 && g.gshift == 7 && g.scale_dtype == XQ_SCALE_BF16 && nj == NJ && (NJ & 3) == 0 && (g.K & 511) == 0 &&
                    (ks & 511) == 0 && ((uintptr_t)g.scales & 7) == 0;
    u32x2 scv[I4 ? R : 1][I4 ? G : 1][I4 ? (NJ + 3) / 4 : 1];
    // nvfp4 with e4m3 block scales and nf4 (fp32, group 64) hold 8 scale bytes per row and step, two of them (nf4: one fp32)
    // for each of the row's four lanes.  Lane kq fetches the 8 bytes of step 4 q + kq -- one load per four steps -- and the four
    // lanes of a row then exchange: a 4 x 4 transpose over the wave's four 16-lane rows leaves each lane with its own piece
    // of each of the four steps.
    constexpr bool P8 = FMT == XQ_FMT_NVFP4 || FMT == XQ_FMT_NF4;
    const bool vs4 = P8 && (FMT == XQ_FMT_NF4 || g.scale_dtype == XQ_SCALE_E4M3) && ((uintptr_t)g.scales & 7) == 0;
    u32x2 scx[P8 ? R : 1][P8 ? G : 1][P8 ? (NJ + 3) / 4 : 1];
    uint32_t sx[P8 ? G : 1][4];        // this lane's scale piece for each step of the current group of four
    const uint8_t* wp[G];
    int64_t erow[G];                            // element index of (row, k0 + (EPS / 4) kq), for the per-row scales
#pragma unroll
    for (int gi = 0; gi < G; ++gi) {
        int n = n0 + gi * 16 + rn;
        n = n < nlim ? n : nlim - 1;
        erow[gi] = (int64_t)n * g.K + k0 + kq * (EPS / 4);
        wp[gi] = g.packed + ((int64_t)n * g.K + k0) / EB + kq * 16;
    }
    const int scols = (g.K + 127) >> 7;
    const int64_t round_bytes = (int64_t)rstride * g.K / EB;         // from a round's rows to the next round's
    auto load_step = [&](int t) {
        {
            const int rr = t / NJ, jj = t % NJ, j = t % DJ;
            const int jc = jj < nj ? jj : nj - 1;
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
                w[j][gi] = *(const u32x4*)(wp[gi] + rr * round_bytes + jc * 64);
                if (FMT == XQ_FMT_FP8) {
                    // one scale per 128 x 128 block: the same for the 16 rows of a group and the 64 elements of a step
                    const int nb = n0 + rr * rstride + gi * 16 < g.N ? n0 + rr * rstride + gi * 16 : g.N - 16;
                    sc[j][gi][0] = ((const __attribute__((address_space(4))) uint32_t*)g.scales)[(nb >> 7) * scols + ((k0 + jc * 64) >> 7)];
                } else if (FMT == XQ_FMT_INT4) {
                    if (vs) {
                        if (jj % 4 == 0)
                            scv[I4 ? rr : 0][I4 ? gi : 0][I4 ? jj / 4 : 0] =
                                *(const u32x2*)((const uint16_t*)g.scales + ((erow[gi] + rr * round_bytes * EB) >> 7) + jj);
                    } else {
                        const int64_t si = (erow[gi] + rr * round_bytes * EB + jc * EPS) >> g.gshift;      // group % 32 == 0: one scale per load
                        sc[j][gi][0] = g.scale_dtype == XQ_SCALE_F32 ? ((const uint32_t*)g.scales)[si] : (uint32_t)((const uint16_t*)g.scales)[si] << 16;
                    }
                } else if (vs4) {
                    // (byte offset of a row's scales = element index / 16 in both formats; steps past the last are clamped onto it)
                    if (jj % 4 == 0) {
                        const int js = jj + kq < nj ? jj + kq : nj - 1;
                        scx[P8 ? rr : 0][P8 ? gi : 0][P8 ? jj / 4 : 0] =
                            *(const u32x2*)(g.scales + (((erow[gi] & ~(int64_t)127) + rr * round_bytes * EB + (int64_t)js * EPS) >> 4));
                    }
                } else if (FMT == XQ_FMT_NF4) {
                    sc[j][gi][0] = ((const uint32_t*)g.scales)[(erow[gi] + rr * round_bytes * EB + jc * EPS) >> 6];       // fp32, group 64
                } else {
                    const int64_t si = (erow[gi] + rr * round_bytes * EB + jc * EPS) >> 4;         // two blocks of 16 per load
                    if (g.scale_dtype == XQ_SCALE_E4M3) {
                        sc[j][gi][0] = *(const uint16_t*)(g.scales + si);
                        sc[j][gi][1] = 0;
                    } else {
                        const u32x2 t = *(const u32x2*)((const uint32_t*)g.scales + si);
                        sc[j][gi][0] = t[0];
                        sc[j][gi][1] = t[1];
                    }
                }
            }
        }
    };
#pragma unroll
    for (int t = 0; t < DJ; ++t) load_step(t);
    __builtin_amdgcn_sched_barrier(0);
    // (PRE: the arguments the loads above need arrived in registers with the wave; the others are fetched now, in one go)
    if constexpr (PRE)
        asm volatile("" ::"s"(g.global_scale), "s"(g.lora_B), "s"(g.r), "s"(g.su_scale), "s"(g.bias), "s"(g.y), "s"(g.ldy), "s"(g.spin_limit));

    // ---- x slice -> LDS (the wave's own area; LDS operations of one wave execute in order, no barrier)
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < XC; ++c)
            if (i < g.M && c * 64 + lane < ppr) *(u32x4*)(slab + i * XP + (c * 64 + lane) * 16) = xr[i][c];
    float* nf4_lds = (float*)(slab + g.slab - 64);          // 16 levels at the end of the wave's area
    if (FMT == XQ_FMT_NF4 && lane < 16) nf4_lds[lane] = kNf4Level[lane];
    __builtin_amdgcn_sched_barrier(0);

    // ---- what the finish needs is requested behind the last weight load (loads return in order, and wave 0's read of the
    // launch count is slow): the block's rows of B (thread t < 384: row t / 4, ranks 4 (t % 4) ..), the bias of column
    // tid % 64 of each round, `gen`
    const int nl = tid & 63;
    f32x4 bq = {0.0f, 0.0f, 0.0f, 0.0f};
    const int brow = tid >> 2, bpiece = tid & 3;
    const int brow_n = n0 + (brow / (16 * G)) * rstride + brow % (16 * G);     // the weight row of the block's row `brow`
    const bool bvalid = lora && brow < 16 * G * R && brow_n < g.N && 4 * bpiece < g.r;
    float bias_v[R];
    auto finish_loads = [&]() {
        const int64_t bn = brow_n < g.N ? brow_n : g.N - 1;
        const float* bp = lora ? g.lora_B + bn * g.r + (4 * bpiece < g.r ? 4 * bpiece : 0) : (const float*)g.x;
        bq = *(const f32x4*)bp;
#pragma unroll
        for (int rr = 0; rr < R; ++rr) {
            const int nfin = (nl < 16 * G && n0 + rr * rstride + nl < g.N) ? n0 + rr * rstride + nl : g.N - 1;
            bias_v[rr] = bf16_to_f32((g.bias ? g.bias : g.x)[g.bias ? nfin : 0]);
        }
        if (lora && wave == 0) gen = __hip_atomic_load(ctl, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    };
    if (T == DJ) finish_loads();
    __builtin_amdgcn_sched_barrier(0);

    // ---- decode + multiply, D[n][m] += deq(W)[n][k] x[m][k], in the order the weights arrive
    const float gsc = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;
    const int xm = rn < g.M ? rn : g.M - 1;
    const unsigned char* xrow = slab + xm * XP + kq * (EPS / 2);
    f32x4 acc[R * G];
#pragma unroll
    for (int gi = 0; gi < R * G; ++gi) acc[gi] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int t = 0; t < T; ++t) {
        const int rr = t / NJ, j = t % NJ, sl = t % DJ;
        if (j < nj) {      // wave-uniform
            bf16x8 xf[MPS];
#pragma unroll
            for (int c = 0; c < MPS; ++c) xf[c] = *(const bf16x8*)(xrow + j * (EPS * 2) + c * 16);
            if constexpr (P8) {
                if (vs4 && j % 4 == 0) {
                    // register k of lane row r <- what lane row k fetched for lane row r: upper / lower halves of the wave swap
                    // between registers two apart (v_permlane32_swap), then odd / even 16-lane rows between neighbours
                    // (v_permlane16_swap)
#pragma unroll
                    for (int gi = 0; gi < G; ++gi) {
                        const u32x2 d = scx[rr][gi][j / 4];
                        uint32_t x0 = d[0], x1 = FMT == XQ_FMT_NF4 ? d[0] : d[0] >> 16, x2 = d[1], x3 = FMT == XQ_FMT_NF4 ? d[1] : d[1] >> 16;
                        const auto p02 = __builtin_amdgcn_permlane32_swap(x0, x2, false, false);
                        const auto p13 = __builtin_amdgcn_permlane32_swap(x1, x3, false, false);
                        const auto q01 = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
                        const auto q23 = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
                        sx[gi][0] = q01[0]; sx[gi][1] = q01[1]; sx[gi][2] = q23[0]; sx[gi][3] = q23[1];
                    }
                }
            }
#pragma unroll
            for (int gi = 0; gi < G; ++gi) {
#pragma unroll
                for (int c = 0; c < MPS; ++c) {
                    bf16x8 wf;
                    if (FMT == XQ_FMT_FP8) {
                        wf = decode8<FMT>(w[sl][gi][2 * c], w[sl][gi][2 * c + 1], __uint_as_float(sc[sl][gi][0]), 0.0f);
                    } else if (FMT == XQ_FMT_INT4) {
                        float sv;
                        if (vs) {
                            const uint32_t v = scv[I4 ? rr : 0][I4 ? gi : 0][I4 ? j / 4 : 0][(j >> 1) & 1];
                            sv = __uint_as_float((j & 1) ? (v & 0xffff0000u) : (v << 16));
                        } else {
                            sv = __uint_as_float(sc[sl][gi][0]);
                        }
                        wf = decode8<FMT>(w[sl][gi][c], 0u, sv, -8.0f * sv);
                    } else if (FMT == XQ_FMT_NF4) {
                        uint32_t sb;
                        if (vs4) sb = sx[P8 ? gi : 0][j & 3];
                        else sb = sc[sl][gi][0];
                        wf = decode8<FMT>(w[sl][gi][c], 0u, __uint_as_float(sb), 0.0f, nf4_lds);
                    } else {
                        float sv;   // block c / 2 of the load's two
                        if (vs4) sv = e4m3_to_f32((uint8_t)(sx[P8 ? gi : 0][j & 3] >> (8 * (c >> 1))));
                        else if (g.scale_dtype == XQ_SCALE_E4M3) sv = e4m3_to_f32((uint8_t)(sc[sl][gi][0] >> (8 * (c >> 1))));
                        else sv = __uint_as_float(sc[sl][gi][c >> 1]);
                        wf = decode8<FMT>(w[sl][gi][c], 0u, sv * gsc, 0.0f);
                    }
                    acc[rr * G + gi] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, xf[c], acc[rr * G + gi], 0, 0, 0);
                }
            }
        }
        if (t + DJ < T) load_step(t + DJ);              // this step's registers are free
        if (t + DJ + 1 == T) finish_loads();
        __builtin_amdgcn_sched_barrier(0);
    }

    // this block may be counted once its reads of `gen` have returned: wave 0's has, like the weights requested before it;
    // in a block that forms an su part wave 4 has read it too and says so when it has published
    if (lora && wave == 0) {
        bool publisher_done = true;
        if (su_block) {
            int spins = 0;
            while (!(publisher_done = __hip_atomic_load(su_flag + 4, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != 0) && spins < g.spin_limit) {
                __builtin_amdgcn_s_sleep(2);
                ++spins;
            }
        }
        // (a block whose publishing wave is that late is never counted: the closer then gives up and marks the slot failed)
        if (lane == 0 && publisher_done) count_block();
    }

    // ---- the wave's sums -> its own LDS area (its x slice is no longer needed): tile gi, register q, lane; B rows -> LDS
    float* part = (float*)slab;
#pragma unroll
    for (int gi = 0; gi < R * G; ++gi)
#pragma unroll
        for (int q = 0; q < 4; ++q) part[gi * 256 + q * 64 + lane] = acc[gi][q];
    if (tid < 384) *(f32x4*)(b_tile + brow * 20 + bpiece * 4) = bvalid ? bq : f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // ---- wave 0 (its loads were requested first, so it gets here first) collects the su parts while the other waves are
    // still streaming: entry q * 64 + l of a part is su[j = 4 (l >> 4) + q][m = l & 15]
    if (lora && wave == 0) {
        const bool closer = bx == nb - 1;      // this block moves the launch count on
        float s[4];
        int spins = 0;
        const bool failed_slot = gen == kGenPoison;
        bool missing = failed_slot, open = closer && !failed_slot;
        if (!failed_slot) do {
#pragma unroll
            for (int q = 0; q < 4; ++q) s[q] = 0.0f;
            missing = false;
            uint32_t started = 0;       // lane l < 32: copy l
            if (open && lane < kCtlCopies)
                started = __hip_atomic_load(g.slot + kSlotCtl + (kCtlCopies + lane) * kCtlStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            for (int p0 = 0; p0 < g.nsu; p0 += 8) {
                // The first look goes through the caches: the 32 blocks of an XCD then share one fetch of each line, where
                // 256 blocks' reads past the caches of the same few lines would queue at their memory channels for
                // microseconds and hold up the weight stream.  What a cached look returns is still judged entry by
                // entry by its tag; a second look is needed only if this one came before the parts, and goes to memory.
                uint64_t t[8][4];
                if (spins == 0) {
#pragma unroll
                    for (int u = 0; u < 8; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            t[u][q] = __hip_atomic_load((const uint64_t*)g.slot + (p0 + u < g.nsu ? p0 + u : g.nsu - 1) * 256 + q * 64 + lane,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                } else {
#pragma unroll
                    for (int u = 0; u < 8; ++u)
#pragma unroll
                        for (int q = 0; q < 4; ++q)
                            t[u][q] = __hip_atomic_load((const uint64_t*)g.slot + (p0 + u < g.nsu ? p0 + u : g.nsu - 1) * 256 + q * 64 + lane,
                                                        __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
#pragma unroll
                for (int u = 0; u < 8; ++u)
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        missing |= (uint32_t)(t[u][q] >> 32) != gen + 1;
                        s[q] += p0 + u < g.nsu ? __uint_as_float((uint32_t)t[u][q]) : 0.0f;
                    }
            }
            missing = __any(missing);
            if (open) {
#pragma unroll
                for (int d = 32; d >= 1; d >>= 1) started += __shfl_xor(started, d, 64);
                if (started == (uint32_t)nb) {
                    // every block has read `gen`: the next launch counts from gen + 1
                    if (lane < kCtlCopies) {
                        __hip_atomic_store(g.slot + kSlotCtl + lane * kCtlStride, gen + 1 == kGenPoison ? 0u : gen + 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(g.slot + kSlotCtl + (kCtlCopies + lane) * kCtlStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    open = false;
                }
            }
            if (missing || open) {
                __builtin_amdgcn_s_sleep(8);
                ++spins;
            }
        } while ((missing || open) && spins < g.spin_limit);
        // A closer that gave up cannot tell which blocks have yet to read the launch count, so no value it could store
        // would keep this launch's late parts and the next launch's apart.  It marks the slot failed instead: every block
        // that reads the mark (late blocks of this launch, all blocks of later launches) publishes nothing and writes
        // NaN, until the host clears the library's slots (reset_skinny_rows_slots).  Never values from stale sums.
        if (open && lane < kCtlCopies)
            __hip_atomic_store(g.slot + kSlotCtl + lane * kCtlStride, kGenPoison, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // a block that is about to write NaN says so where the host can see it (no return value asked for)
        if ((missing || open) && lane == 0) __hip_atomic_fetch_add(g.fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int j = 4 * (lane >> 4) + q, m = lane & 15;
            su_tot[m * 16 + j] = j < g.r ? s[q] * g.su_scale : 0.0f;
        }
        if (lane == 0) ((int*)su_tot)[256] = (missing || open) ? 0 : 1;
    }
    lds_barrier();

    // ---- outputs: thread (nl, mg) finishes y[mg][n] and y[mg + 8][n] for row n = n0 + 16 G rr + nl of every round: the eight
    // waves' sums in wave order, the low-rank term rank by rank in fp32, the bias, one rounding
    const int mg = tid >> 6;
    const int gi_f = nl >> 4, nloc = nl & 15;
    const bool ok = !lora || ((const int*)su_tot)[256] != 0;
    float gate_v[2] = {0.0f, 0.0f};                     // GU: the rounded gate outputs of round 0, until round 1 has the up outputs
#pragma unroll
    for (int rr = 0; rr < R; ++rr) {
        const int nrow = rr * 16 * G + nl;              // row of the block
        const bool nvalid = nl < 16 * G && n0 + rr * rstride + nl < g.N && n0 + nl < nlim;
        f32x4 bv[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) bv[q] = *(const f32x4*)(b_tile + (nl < 16 * G ? nrow : 0) * 20 + 4 * q);
#pragma unroll
        for (int mm = 0; mm < 2; ++mm) {
            const int m = mg + 8 * mm;
            if (m < g.M && nvalid) {
                // D[nloc][m] of a wave's tile sits in register nloc & 3 of lane 16 (nloc >> 2) + m
                const int idx = (rr * G + gi_f) * 256 + (nloc & 3) * 64 + (nloc >> 2) * 16 + m;
                float o = 0.0f;
#pragma unroll
                for (int ww = 0; ww < 8; ++ww) o += ((const float*)(smem + ww * g.slab))[idx];
                if (lora) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x4 sv = *(const f32x4*)(su_tot + m * 16 + 4 * q);
#pragma unroll
                        for (int c = 0; c < 4; ++c) o = __builtin_fmaf(sv[c], bv[q][c], o);
                    }
                }
                if (g.bias) o += bias_v[rr];
                if (!ok) o = __builtin_nanf("");
                if constexpr (GU) {
                    if (rr == 0) gate_v[mm] = round_bf16(o);
                    else g.y[(int64_t)m * g.ldy + n0 + nl] = to_bf16(round_bf16(gate_v[mm] * sigmoid_f32(gate_v[mm])) * round_bf16(o));
                } else {
                    g.y[(int64_t)m * g.ldy + n0 + nrow] = to_bf16(o);
                }
            }
        }
    }
}


template <int FMT, int G, int NJ, int MR, int R>
__global__ void __launch_bounds__(512, 1) skinny_rows_kernel(SkinnyRowsArgs g) {
    skinny_rows_body<FMT, G, NJ, MR, R>(g, (int)blockIdx.x, (int)gridDim.x);
}

// The same kernel with the arguments its first loads need as leading scalars: the hardware hands a kernel's first 16
// argument dwords to each wave in registers (where the platform supports it; otherwise they are fetched like the rest),
// so the wave's first loads do not wait for a round trip to the argument block.
template <int FMT, int G, int NJ, int MR, int R, bool GU = false>
__global__ void __launch_bounds__(512, 1) skinny_rows_kernel_p(const bf16_t* x, int32_t ldx, int32_t M, int32_t N, int32_t K,
                                                               const uint8_t* packed, const uint8_t* scales, uint32_t* slot,
                                                               const float* lora_A, int32_t nsu, int32_t fmt_bits, SkinnyRowsArgs rest) {
    SkinnyRowsArgs g = rest;
    g.x = x; g.ldx = ldx; g.M = M; g.N = N; g.K = K; g.packed = packed; g.scales = scales; g.slot = slot; g.lora_A = lora_A;
    g.nsu = nsu; g.gshift = fmt_bits & 255; g.scale_dtype = fmt_bits >> 8;
    g.xpitch = (K >> 3) * 2 + 16;
    int slab = M * g.xpitch + 64;
    slab = slab < (G * R + 1) * 1024 ? (G * R + 1) * 1024 : slab;
    g.slab = (slab + 15) & ~15;
    skinny_rows_body<FMT, G, NJ, MR, R, true, GU>(g, (int)blockIdx.x, (int)gridDim.x);
}

// Several forwards that share x (and format, K and M) in one launch: the grid is the forwards' grids one after the other,
// each forward with its own weight, factors, outputs and slot; a block finds its forward by its index.
constexpr int kRowsMaxJobs = 4;
struct SkinnyRowsBatch {
    SkinnyRowsArgs job[kRowsMaxJobs];
    int32_t first[kRowsMaxJobs + 1];    // first block of each forward; entries past the last forward hold the grid size
};
// (the boundaries between the forwards are leading scalars, with the wave from the start: the one fetch of the block's own
// argument set does not wait for another fetch to tell it which set that is)
template <int FMT, int G, int NJ, int MR, int R>
__global__ void __launch_bounds__(512, 1) skinny_rows_multi_kernel(int32_t first1, int32_t first2, int32_t first3, int32_t first4,
                                                                   SkinnyRowsBatch b) {
    const int bx = (int)blockIdx.x;
    const int i = (bx >= first1 ? 1 : 0) + (bx >= first2 ? 1 : 0) + (bx >= first3 ? 1 : 0);   // uniform
    const int lo = i == 0 ? 0 : i == 1 ? first1 : i == 2 ? first2 : first3;
    const int hi = i == 0 ? first1 : i == 1 ? first2 : i == 2 ? first3 : first4;
    skinny_rows_body<FMT, G, NJ, MR, R>(b.job[i], bx - lo, hi - lo);
}

// ---- slots: device memory that belongs to the library (zero when the code object is loaded).
// Each device holds its own copy of the array at its own address, reached through hipGetSymbolAddress with that device
// current.  A slot is tied to the caller's scratch pointer, so calls that may legally overlap (different workspaces)
// never share one.  A slot changes hands only when nothing can still refer to it: a slot used by a launch that was
// recorded into a HIP graph stays with its key for good (the graph holds its address), and another slot is taken over
// only once the stream of its last launch has run dry.  When no slot can be had that way the caller takes the
// two-launch organisation, which needs none.  The word behind the slots counts the blocks whose bounded wait gave up.
static __device__ __align__(256) uint32_t rows_slots[kSlots * kSlotWords + 64];

namespace {
constexpr int kMaxDevices = 64;
struct SlotHost {
    const void* key;
    uint64_t used;          // 0: never used
    hipStream_t stream;     // stream of the last launch through the slot
    bool pinned;            // a captured launch refers to it
};
std::mutex g_slots_mu;
uint32_t* g_slots_ptr[kMaxDevices] = {};
SlotHost g_slot[kMaxDevices][kSlots] = {};
uint64_t g_slot_clock = 0;
}  // namespace

// looks of a bounded wait before it gives up: a process-wide test switch (a small value forces the give-up paths, in which
// every kernel still ends and the outputs concerned are NaN)
static std::atomic<int> g_rows_spin_limit{kRowsSpinLimit};
void set_skinny_rows_spin_limit(int limit) { g_rows_spin_limit = limit > 0 ? limit : kRowsSpinLimit; }

// the slot array of the current device (address resolved once per device); g_slots_mu held by the caller
static int rows_slots_base(int* dev_out, uint32_t** base) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        xq_set_error("xq_linear_fwd: cannot identify the current device: %s", hipGetErrorString(e));
        return XQ_ERR_LAUNCH;
    }
    if (!g_slots_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(rows_slots));
        if (e != hipSuccess || !p) {
            xq_set_error("xq_linear_fwd: hipGetSymbolAddress(rows_slots) failed on device %d: %s", dev, hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        g_slots_ptr[dev] = (uint32_t*)p;
    }
    *dev_out = dev;
    *base = g_slots_ptr[dev];
    return XQ_OK;
}

// The slot of `key` on the current device for a launch on `stream`, and the device's failure counter.
// XQ_ERR_UNSUPPORTED (no message): every slot belongs to another key and none of them can be shown to be idle.
static int rows_slot(const void* key, hipStream_t stream, uint32_t** out, uint32_t** fail) {
    std::lock_guard<std::mutex> lock(g_slots_mu);
    int dev = 0;
    uint32_t* base = nullptr;
    int rc = rows_slots_base(&dev, &base);
    if (rc) return rc;
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cap) != hipSuccess) {
        (void)hipGetLastError();
        cap = hipStreamCaptureStatusNone;
    }
    const bool capturing = cap != hipStreamCaptureStatusNone;
    SlotHost* tab = g_slot[dev];
    int s = -1;
    for (int i = 0; i < kSlots && s < 0; ++i)
        if (tab[i].used && tab[i].key == key) s = i;
    for (int i = 0; i < kSlots && s < 0; ++i)
        if (!tab[i].used) s = i;
    if (s < 0) {
        // Least recently used first.  A slot whose last launch went to this same stream can be taken over at once: the
        // stream runs its launches one after the other.  One last used on another stream only when that stream has run
        // dry (a host-side look, no work is enqueued; not while capturing: queries are not capture-safe everywhere).
        for (int tries = 0; tries < 8 && s < 0; ++tries) {
            int oldest = -1;
            for (int i = 0; i < kSlots; ++i)
                if (!tab[i].pinned && (oldest < 0 || tab[i].used < tab[oldest].used)) oldest = i;
            if (oldest < 0) break;
            if (tab[oldest].stream == stream) {
                s = oldest;
            } else if (!capturing) {
                const hipError_t q = hipStreamQuery(tab[oldest].stream);
                if (q == hipSuccess) s = oldest;
                else if (q != hipErrorNotReady) (void)hipGetLastError();
            }
            if (s < 0) tab[oldest].used = ++g_slot_clock;      // busy elsewhere: look at the next oldest
        }
    }
    if (s < 0) return XQ_ERR_UNSUPPORTED;
    tab[s].key = key;
    tab[s].used = ++g_slot_clock;
    tab[s].stream = stream;
    tab[s].pinned = tab[s].pinned || capturing;
    *out = base + (size_t)s * kSlotWords;
    *fail = base + (size_t)kSlots * kSlotWords;
    return XQ_OK;
}

// Clears the slots of the current device (launch counts, marks of failed waits, published parts, the failure count): for
// a host that has seen NaN outputs after a forced or real give-up.  Waits for the device before and after; no forward may
// be in flight, and graphs that captured a one-launch forward keep their slots' addresses (the cleared slot works on).
int reset_skinny_rows_slots() {
    std::lock_guard<std::mutex> lock(g_slots_mu);
    int dev = 0;
    uint32_t* base = nullptr;
    int rc = rows_slots_base(&dev, &base);
    if (rc) return rc;
    hipError_t e = hipDeviceSynchronize();
    if (e == hipSuccess) e = hipMemset(base, 0, sizeof(uint32_t) * ((size_t)kSlots * kSlotWords + 64));
    if (e == hipSuccess) {
        for (int i = 0; i < kSlots; ++i)
            if (!g_slot[dev][i].pinned) g_slot[dev][i] = SlotHost{};
    }
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        xq_set_error("xq_skinny_reset: %s", hipGetErrorString(e));
        return XQ_ERR_LAUNCH;
    }
    return XQ_OK;
}

// What the one-launch forwards of the current device have reported since the last call: blocks whose bounded wait gave up
// (each wrote NaN outputs) and slots marked failed (every forward through such a slot writes NaN).  Waits for `stream`,
// reads a few words back, and, when anything was found, waits for the whole device, clears the marks and the count, so
// that later forwards are exact again.  Costs one stream synchronisation: for the points where the host waits anyway.
int skinny_rows_status(int* gave_up, int* failed_slots, hipStream_t stream) {
    *gave_up = 0;
    *failed_slots = 0;
    std::lock_guard<std::mutex> lock(g_slots_mu);
    int dev = 0;
    uint32_t* base = nullptr;
    int rc = rows_slots_base(&dev, &base);
    if (rc) return rc;
    uint32_t count = 0, gens[kSlots];
    hipError_t e = hipStreamSynchronize(stream);
    if (e == hipSuccess) e = hipMemcpy(&count, base + (size_t)kSlots * kSlotWords, 4, hipMemcpyDeviceToHost);
    if (e == hipSuccess)
        e = hipMemcpy2D(gens, 4, base + kSlotCtl, sizeof(uint32_t) * (size_t)kSlotWords, 4, kSlots, hipMemcpyDeviceToHost);
    int bad = 0;
    if (e == hipSuccess) {
        for (int i = 0; i < kSlots; ++i) bad += gens[i] == kGenPoison;
        if (bad || count) {
            e = hipDeviceSynchronize();
            for (int i = 0; i < kSlots && e == hipSuccess; ++i)
                if (gens[i] == kGenPoison)      // the whole slot: parts of the failed launch must not meet a launch count that starts over
                    e = hipMemset(base + (size_t)i * kSlotWords, 0, sizeof(uint32_t) * (size_t)kSlotWords);
            if (e == hipSuccess) e = hipMemset(base + (size_t)kSlots * kSlotWords, 0, 4);
            if (e == hipSuccess) e = hipDeviceSynchronize();
        }
    }
    if (e != hipSuccess) {
        xq_set_error("xq_skinny_status: %s", hipGetErrorString(e));
        return XQ_ERR_LAUNCH;
    }
    *gave_up = (int)(count > 0x7fffffffu ? 0x7fffffffu : count);
    *failed_slots = bad;
    return XQ_OK;
}

// geometry of a launch: NJ bound and row groups per block
struct RowsPlan { int nj, njt, G, R, MR, xpitch, slab; size_t lds; };
static bool rows_plan_multi(const xq_weight* const* ws, int n_w, int64_t M, RowsPlan* p);
static bool rows_plan(const xq_weight* w, int64_t M, RowsPlan* p) { return rows_plan_multi(&w, 1, M, p); }
// one geometry for several weights of one format and K that share a launch: each weight's rows are whole blocks
static bool rows_plan_multi(const xq_weight* const* ws, int n_w, int64_t M, RowsPlan* p) {
    const xq_weight* w = ws[0];
    const int64_t K = w->cols;
    const bool f8 = w->format == XQ_FMT_FP8;
    const int eps = f8 ? 64 : 128;
    if (K % (8 * eps) != 0) return false;
    const int ks = (int)(K >> 3);
    p->nj = ks / eps;
    if (f8) p->njt = p->nj <= 4 ? 4 : p->nj <= 8 ? 8 : p->nj <= 16 ? 16 : p->nj <= 24 ? 24 : 0;
    else p->njt = p->nj <= 4 ? 4 : p->nj <= 8 ? 8 : p->nj <= 12 ? 12 : 0;
    if (!p->njt) return false;
    p->MR = M <= 1 ? 1 : M <= 8 ? 8 : 16;
    // x rows in registers: 16 rows only with slices of at most 1 KB, 8 rows with at most 2 KB (register budget)
    if (p->MR == 16 && p->njt * eps > 512) return false;
    if (p->MR == 8 && p->njt * eps > 1024) return false;
    // as many row groups per block as give about one block per compute unit, within 24 loads per lane
    int64_t groups = 0;
    for (int i = 0; i < n_w; ++i) groups += ws[i]->rows / 16;
    const int cus = num_cus();
    int G = (int)((groups + cus - 1) / cus);
    const int gmax = p->njt <= 4 ? 3 : p->njt <= 8 ? (f8 ? 3 : 2) : p->njt <= 12 ? 2 : 1;
    p->G = G < 1 ? 1 : G > gmax ? gmax : G;
    // more blocks than compute units would run one after the other, each with its own start-up and finish (that costs
    // more than the second launch of the other organisation): twice the rows go to one block in two rounds instead,
    // where the shape allows it
    p->R = 1;
    int64_t blocks = 0;
    bool sixes = true;
    for (int i = 0; i < n_w; ++i) {
        blocks += xq_cdiv(ws[i]->rows / 16, p->G);
        sixes = sixes && (ws[i]->rows / 16) % 6 == 0;
    }
    if (blocks > cus) {
        const bool two_rounds = p->G == 3 && p->njt * eps <= 512 && sixes && groups / 6 <= cus;
        if (!two_rounds) return false;
        p->R = 2;
    }
    p->xpitch = ks * 2 + 16;
    int slab = (int)M * p->xpitch + 64;                       // x slice + the NF4 levels
    if (slab < (p->G * p->R + 1) * 1024) slab = (p->G * p->R + 1) * 1024;   // later: the wave's sums
    p->slab = (slab + 15) & ~15;
    p->lds = (size_t)8 * p->slab + 272 * 4 + 96 * 20 * 4 + 4 * 256 * 4 + 64;
    return p->lds <= 160 * 1024;
}

bool skinny_rows_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r) {
    if (M < 1 || M > 16 || w->num_experts != 1 || w->rows % 16 != 0) return false;
    if (w->format != XQ_FMT_FP8 && w->layout != XQ_LAYOUT_FLAT) return false;
    if (w->format == XQ_FMT_NF4 && (w->group != 64 || w->scale_dtype != XQ_SCALE_F32)) return false;
    if (w->format == XQ_FMT_INT4 && (w->group < 32 || (w->group & (w->group - 1)) != 0 ||
                                     (w->scale_dtype != XQ_SCALE_F32 && w->scale_dtype != XQ_SCALE_BF16)))
        return false;
    if (w->format == XQ_FMT_NVFP4 && w->scale_dtype != XQ_SCALE_E4M3 && w->scale_dtype != XQ_SCALE_F32) return false;
    RowsPlan p;
    if (!rows_plan(w, M, &p)) return false;
    if (r > 0) {
        if (lora_dtype != XQ_DT_F32 || r > 16 || r % 4 != 0 || !xq_aligned(lora_A, 16) || !xq_aligned(lora_B, 16)) return false;
        if (w->cols % kSuPartK != 0 || w->cols / kSuPartK > kSuMaxParts) return false;
        if (w->cols / kSuPartK > xq_cdiv(w->rows / 16, p.G * p.R)) return false;   // a block forms at most one su part
    }
    return true;
}

// `batch` == nullptr: the forward `g` alone; otherwise the forwards of `*batch` as one launch
template <int FMT, int G, int NJ, int MR, int R>
static int launch_rows_one(const SkinnyRowsArgs& g, const SkinnyRowsBatch* batch, unsigned grid, size_t lds, hipStream_t s) {
    static std::atomic<bool> attr_set{false};   // per instantiation; the attribute calls are idempotent: a race only repeats them
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)skinny_rows_kernel<FMT, G, NJ, MR, R>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)skinny_rows_multi_kernel<FMT, G, NJ, MR, R>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess)
            e = hipFuncSetAttribute((const void*)skinny_rows_kernel_p<FMT, G, NJ, MR, R>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) {
            xq_set_error("xq_linear_fwd: cannot raise the dynamic LDS limit: %s", hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    // XQ_ROWS_PRELOAD=0 launches the form that fetches every argument itself (A/B measurements)
    static const bool preload = [] { const char* e = getenv("XQ_ROWS_PRELOAD"); return e ? atoi(e) != 0 : true; }();
    if (batch) skinny_rows_multi_kernel<FMT, G, NJ, MR, R><<<grid, 512, lds, s>>>(batch->first[1], batch->first[2], batch->first[3], batch->first[4], *batch);
    else if (preload && g.ldx < (1ll << 31))
        skinny_rows_kernel_p<FMT, G, NJ, MR, R><<<grid, 512, lds, s>>>(g.x, (int32_t)g.ldx, g.M, g.N, g.K, g.packed, g.scales, g.slot, g.lora_A,
                                                                         g.nsu, g.gshift | g.scale_dtype << 8, g);
    else skinny_rows_kernel<FMT, G, NJ, MR, R><<<grid, 512, lds, s>>>(g);
    return XQ_OK;
}

template <int FMT, int G, int NJ, int R>
static int launch_rows_mr(const SkinnyRowsArgs& g, const SkinnyRowsBatch* batch, int MR, unsigned grid, size_t lds, hipStream_t s) {
    constexpr int EPS = FMT == XQ_FMT_FP8 ? 64 : 128;
    if (MR == 1) return launch_rows_one<FMT, G, NJ, 1, R>(g, batch, grid, lds, s);
    if constexpr (NJ * EPS <= 1024) {
        if (MR == 8) return launch_rows_one<FMT, G, NJ, 8, R>(g, batch, grid, lds, s);
    }
    if constexpr (NJ * EPS <= 512) {
        if (MR == 16) return launch_rows_one<FMT, G, NJ, 16, R>(g, batch, grid, lds, s);
    }
    XQ_REQUIRE(false, "xq_linear_fwd: internal error: no one-launch skinny kernel for %d x rows, %d steps", MR, NJ);
}

template <int FMT>
static int launch_rows_fmt(const SkinnyRowsArgs& g, const SkinnyRowsBatch* batch, const RowsPlan& p, unsigned grid, hipStream_t s) {
    constexpr int EPS = FMT == XQ_FMT_FP8 ? 64 : 128;
#define XQ_ROWS_CASE(GG, NN, RR) \
    if (p.G == GG && p.njt == NN && p.R == RR) return launch_rows_mr<FMT, GG, NN, RR>(g, batch, p.MR, grid, p.lds, s)
    XQ_ROWS_CASE(1, 4, 1); XQ_ROWS_CASE(2, 4, 1); XQ_ROWS_CASE(3, 4, 1); XQ_ROWS_CASE(3, 4, 2);
    XQ_ROWS_CASE(1, 8, 1); XQ_ROWS_CASE(2, 8, 1);
    if constexpr (FMT == XQ_FMT_FP8) {
        XQ_ROWS_CASE(3, 8, 1); XQ_ROWS_CASE(3, 8, 2); XQ_ROWS_CASE(1, 16, 1); XQ_ROWS_CASE(1, 24, 1);
    } else {
        XQ_ROWS_CASE(1, 12, 1); XQ_ROWS_CASE(2, 12, 1);
    }
#undef XQ_ROWS_CASE
    (void)EPS;
    XQ_REQUIRE(false, "xq_linear_fwd: internal error: no one-launch skinny kernel for %d row groups, %d steps, %d rounds", p.G, p.njt, p.R);
}

static int rows_args(const xq_weight* w, const RowsPlan& p, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                     int r, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, const void* slot_key, hipStream_t stream,
                     SkinnyRowsArgs* out) {
    SkinnyRowsArgs& g = *out;
    g.x = x; g.ldx = ldx; g.M = (int)M; g.N = (int)w->rows; g.K = (int)w->cols;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.gshift = 0;
    for (int v = w->group; v > 1; v >>= 1) ++g.gshift;
    g.scale_dtype = w->scale_dtype;
    g.lora_A = (const float*)lora_A; g.lora_B = (const float*)lora_B; g.r = r; g.su_scale = scaling;
    g.bias = bias; g.y = y; g.ldy = ldy;
    g.xpitch = p.xpitch; g.slab = p.slab;
    g.nsu = r > 0 ? (int)(w->cols / kSuPartK) : 0;
    g.slot = nullptr;
    g.spin_limit = g_rows_spin_limit.load();
    g.fail = nullptr;
    if (r > 0) return rows_slot(slot_key, stream, &g.slot, &g.fail);
    return XQ_OK;
}

int launch_skinny_rows(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B, int r,
                       float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, const void* slot_key, hipStream_t stream) {
    if (skinny_gemv_supported(w, M, lora_A, lora_B, XQ_DT_F32, r)) return launch_skinny_gemv(w, x, lora_A, lora_B, r, scaling, bias, y, slot_key, stream, false);
    RowsPlan p;
    XQ_REQUIRE(rows_plan(w, M, &p), "xq_linear_fwd: internal error: shape not supported by the one-launch skinny kernel");
    SkinnyRowsArgs g;
    const int rc = rows_args(w, p, x, ldx, M, lora_A, lora_B, r, scaling, bias, y, ldy, slot_key, stream, &g);
    if (rc) return rc;
    const unsigned grid = (unsigned)xq_cdiv(w->rows / 16, p.G * p.R);
    switch (w->format) {
        case XQ_FMT_FP8: return launch_rows_fmt<XQ_FMT_FP8>(g, nullptr, p, grid, stream);
        case XQ_FMT_INT4: return launch_rows_fmt<XQ_FMT_INT4>(g, nullptr, p, grid, stream);
        case XQ_FMT_NF4: return launch_rows_fmt<XQ_FMT_NF4>(g, nullptr, p, grid, stream);
        default: return launch_rows_fmt<XQ_FMT_NVFP4>(g, nullptr, p, grid, stream);
    }
}

// ---------------------------------------------------------------- M = 1, every format: dot products instead of MFMA tiles
// One token against a packed weight needs no matrix cores, and the organisation above -- 8 waves per CU, a load instruction
// that takes 64 bytes of each of 16 rows -- is what keeps it from the rate of a plain read when the bytes come from HBM
// (8 waves per CU pull at most ~6 TB/s however deep their queues; a linear read by 32 waves per CU reaches 6.9).  Here the
// waves stream 1 KB pieces of whole rows: a row is shared by K / 1024 waves (a "set"; wave w of it owns the bytes 1024 w ..
// of every row the set works on, so a load instruction is one contiguous KB of one row), rows go through a set in groups of
// RB, the next group's RB loads of a lane in flight while it works on the current one.  A lane decodes its 16 weights (fp8) of a
// row to the reference decoder's bf16 values (decode8) and multiplies them with its x elements -- the same for every row,
// held in registers as bf16 pairs -- by v_dot2c_f32_bf16 (exact products, fp32 sums); the lanes' sums of a row meet by
// lane-permuting adds, the waves' through LDS in wave order.
// A block is as many sets as make up to 8 waves, two blocks to a CU, plus one more wave that does not stream: it takes the
// block's part in the low-rank exchange (the slots and the launch-count protocol of the kernel above: parts of z = A x
// published with the launch's tag, collected by every block, the last block moves the launch count on), fetches the B rows
// and bias, and finishes the block's rows (at most 64) when the sets are through.  The parts of z (16 ranks x 512 elements
// each) are formed by K / 512 blocks of their own at the head of the grid, which do nothing else and are gone after a few
// microseconds.  So no streaming wave ever waits for anything but its own weights -- under a saturated memory system any
// dependent load costs ~3 us, and a block that is late by that makes the launch late by that -- and the parts of z are
// read once per block: ~500 readers of the same few lines, not thousands.  (A part's entry for rank j sits at pair j of the
// part's 256; tags keep launches of the two kernels on one slot apart.)
// The 4-bit formats take the same kernel with 32 weights per lane and load (rows of 2 KB per wave; nvfp4: the lane's two
// e4m3 block scales come as one word, the tensor's global scale is a scalar; nf4: the 16 levels in a per-wave table in
// LDS).  Their time is the decode's -- as many instructions per weight as block fp8, twice as many per byte.  nvfp4 and nf4
// are ahead of the MFMA kernel on every shape measured (-8 % on many short rows to -30 % on few, nf4 -16 to -34 %); int4 is
// level with it on weights of many short rows (those stay on that kernel) and ahead where that kernel's organisation
// fits badly (q, kv, down: -15 %).  Several forwards on one x (xq_linear_fwd_multi) and gate | up with the SwiGLU finish
// (xq_linear_fwd_swiglu) take the same body: see skinny_gemv_multi_kernel and the GU form below.
constexpr int kGemvRows = 4;                        // rows per group: with the next group's, 8 loads of a lane in flight
constexpr int kGemvSlots = 64 / kGemvRows;          // groups of rows per block at most (all its sets together)

// acc += w.lo * x.lo + w.hi * x.hi on bf16 pairs (exact products, one fp32 sum).  Written as the instruction: the
// compiler's builtin for it, fed with elements of vectors, came out with one register pair for all four pairs of a vector.
__device__ __forceinline__ void dot2_bf16(float& acc, uint32_t w, uint32_t x) {
    asm("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(acc) : "v"(w), "v"(x));
}
// the value of the lane that a DPP control names (all lanes active here)
template <int CTRL>
__device__ __forceinline__ float lane_perm(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// v + the same lanes of the other 16-lane rows: the rows swap in pairs (v_permlane16_swap), then the wave's halves
// (v_permlane32_swap); every lane ends with the sum of the four lanes 16 apart, added as (r0 + r1) + (r2 + r3)
__device__ __forceinline__ float sum_rows_of_16(float v) {
    const uint32_t u = __float_as_uint(v);
    auto p = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float h = __uint_as_float(p[0]) + __uint_as_float(p[1]);
    const uint32_t hu = __float_as_uint(h);
    auto q = __builtin_amdgcn_permlane32_swap(hu, hu, false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}
__device__ __forceinline__ float read_lane(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }

struct GemvArgs {
    const bf16_t* x;
    int32_t N, K;
    const uint8_t* packed;
    const uint8_t* scales;         // fp8: fp32 [ceil(N / 128), ceil(K / 128)]; int4: one per group along K; nvfp4: e4m3, one per 16
    const float* global_scale;     // nvfp4: the tensor's second-level scale
    int32_t gshift, scale_dtype;   // int4: log2 of the group size, the scales' type
    const float* lora_A;           // [r, K] fp32
    const float* lora_B;           // [N, r] fp32
    int32_t r;
    float su_scale;
    const bf16_t* bias;
    bf16_t* y;
    int32_t nsu;                   // parts of z (K / 512), 0 without a low-rank term
    int32_t nw, sets, gmax, rps;   // waves of a set, sets of a block, groups of a set at most (sets * gmax <= kGemvSlots), rows of a set
    uint32_t* slot;
    int32_t spin_limit;
    uint32_t* fail;
};

// (registers held to what lets 6 waves share a SIMD: left to itself the compiler spends the 128 that blocks of up to 16 waves
// allow on decoding all rows of a group at once)
// `blk` of `nb`: this block among those of its forward (a launch may hold several forwards, one after the other).
// GU: the weight is gate | up stacked, [2 I, K]; the rows are walked as gate 0, up 0, gate 1, up 1, ... so that the two
// rows of a column meet in neighbouring lanes of the finish, which writes h [I] = bf16(bf16(silu(gate)) * up) from the two
// rounded outputs (the arithmetic of the SwiGLU kernel, ops/fused_silu_and_mul.py:22-60) instead of the outputs themselves.
template <int FMT, int RB, bool GU>
__device__ __forceinline__ void skinny_gemv_body(const GemvArgs& g, const int blk, const int nb) {
    constexpr bool F8 = FMT == XQ_FMT_FP8, NV = FMT == XQ_FMT_NVFP4, NF = FMT == XQ_FMT_NF4;
    constexpr int EPL = F8 ? 16 : 32;                 // weights of a row per lane (one 16-byte load)
    __shared__ float red[kGemvSlots][RB][16];         // [set * gmax + group of the set][row][wave of the set]
    __shared__ float zpart[16][17];                   // a block that forms a part of z: [k slice][rank]
    __shared__ float nf4_tab[NF ? 16 : 1][16];        // nf4: the 16 levels, a copy per wave (16 banks: any mix of codes reads it at full rate)
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const bool lora = g.nsu > 0;
    // row of the weight for row j of the walk
    auto weight_row = [&](int j) { return GU ? ((j & 1) ? (g.N >> 1) + (j >> 1) : (j >> 1)) : j; };

    // ---- the first K / 512 blocks of a launch with a low-rank term form the parts of z and nothing else (they are gone
    // after a few microseconds; a block that streamed as well would be late by a memory latency under load, and the
    // launch with it): 256 threads contract 512 elements of K for the 16 ranks, thread (slice, rank) a run of 32 elements;
    // the slices are summed in order by the threads of slice 0 and published with the launch's tag
    if (blk < g.nsu) {
        const int part = blk;
        if (wave >= 4) return;
        // (the launch count through this XCD's L2: no line of the slot can be there from before the launch, and within a
        // launch the word changes only after every block has read it; the block is counted in once it has been read)
        uint32_t gen = 0;
        if (wave == 0) {
            gen = __hip_atomic_load(g.slot + kSlotCtl + (part % kCtlCopies) * kCtlStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            if (lane == 0) {
                uint32_t one = 1u;
                asm volatile("" : "+v"(one) : "v"(gen));
                __hip_atomic_fetch_add(g.slot + kSlotCtl + (kCtlCopies + part % kCtlCopies) * kCtlStride, one, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
            }
        }
        const int j = tid & 15, sl = tid >> 4;
        const int kb = part * kSuPartK + sl * 32;
        const float* ap = g.lora_A + (int64_t)(j < g.r ? j : 0) * g.K + kb;
        const bf16_t* xp = g.x + kb;
        float a = 0.0f;
#pragma unroll
        for (int e = 0; e < 32; e += 8) {
            const f32x4 a0 = *(const f32x4*)(ap + e), a1 = *(const f32x4*)(ap + e + 4);
            const u32x4 xx = *(const u32x4*)(xp + e);
            // (the factor rounded to bf16 first, as in the other kernels: exact products, fp32 sums)
            a = __builtin_fmaf(round_bf16(a0[0]), __uint_as_float(xx[0] << 16), a); a = __builtin_fmaf(round_bf16(a0[1]), __uint_as_float(xx[0] & 0xffff0000u), a);
            a = __builtin_fmaf(round_bf16(a0[2]), __uint_as_float(xx[1] << 16), a); a = __builtin_fmaf(round_bf16(a0[3]), __uint_as_float(xx[1] & 0xffff0000u), a);
            a = __builtin_fmaf(round_bf16(a1[0]), __uint_as_float(xx[2] << 16), a); a = __builtin_fmaf(round_bf16(a1[1]), __uint_as_float(xx[2] & 0xffff0000u), a);
            a = __builtin_fmaf(round_bf16(a1[2]), __uint_as_float(xx[3] << 16), a); a = __builtin_fmaf(round_bf16(a1[3]), __uint_as_float(xx[3] & 0xffff0000u), a);
        }
        zpart[sl][j] = j < g.r ? a : 0.0f;
        // (the four waves that are left meet at a named point of their own: the block's other waves have ended)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if (tid < 16) {
            float z = 0.0f;
            for (int q = 0; q < 16; ++q) z += zpart[q][tid];
            if (gen != kGenPoison)                    // a slot that is marked failed gets nothing
                __hip_atomic_store((uint64_t*)g.slot + part * 256 + tid, ((uint64_t)(gen + 1) << 32) | __float_as_uint(z), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }

    const int bx = blk - g.nsu;                      // this block among those that stream
    const int nstream = g.sets * g.nw;                // streaming waves; wave `nstream` is the one that does not stream
    const bool streamer = wave < nstream;
    const int st = wave / g.nw, ws = wave - st * g.nw;
    // set v of the launch's nbs * sets takes the rows v * rps .. (v + 1) * rps - 1, in groups of RB (the last one may be short)

    // (the two kinds of waves go separate ways from here, each with the block's barrier in its own path, so that neither
    // carries the other's registers)
    if (streamer) {
        // (written and read by this wave only: LDS operations of a wave execute in order)
        if (NF && lane < 16) nf4_tab[wave][lane] = kNf4Level[lane];
        const int v = bx * g.sets + st;
        const int row0 = v * g.rps;
        const int nrows = row0 < g.N ? (g.N - row0 < g.rps ? g.N - row0 : g.rps) : 0;
        const int gcount = (nrows + RB - 1) / RB;     // at most gmax (host)
        const int kbase = (ws * 64 + lane) * EPL;     // first element of this lane's piece of a row
        const int sc_cols = (g.K + 127) >> 7;
        const int64_t row_bytes = F8 ? g.K : g.K >> 1;
        // a group's pieces and scales (one scale per lane and row: the lane's elements lie in one 128-block, or in one
        // group of at least 32)
        // (an int4 scale is fetched as the aligned 32-bit word that holds it, fp32 or bf16, and picked apart when it is
        // used: a conversion next to the load would wait for every load in flight)
        const bool s32 = g.scale_dtype == XQ_SCALE_F32;
        // (a row past the set's last one stands for that one: the same lines again, nothing more from memory)
        auto issue = [&](u32x4 (&w)[RB], float (&sc)[RB], int gi) {
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                const int n = weight_row(row0 + (gi * RB + i < nrows ? gi * RB + i : nrows - 1));
                w[i] = __builtin_nontemporal_load((const u32x4*)(g.packed + (int64_t)n * row_bytes + (ws * 64 + lane) * 16));
                if (F8) {
                    sc[i] = ((const float*)g.scales)[(n >> 7) * sc_cols + (kbase >> 7)];
                } else if (NF) {
                    sc[i] = ((const float*)g.scales)[((int64_t)n * g.K + kbase) >> 6];
                } else if (NV) {
                    // (the lane's two e4m3 scales, one per 16 weights, inside the aligned word that holds them)
                    const int64_t si = ((int64_t)n * g.K + kbase) >> 4;
                    sc[i] = *(const float*)(g.scales + (si & ~(int64_t)3));
                } else {
                    const int64_t si = ((int64_t)n * g.K + kbase) >> g.gshift;
                    sc[i] = *(const float*)(g.scales + ((s32 ? si << 2 : si << 1) & ~(int64_t)3));
                }
            }
        };
        // the scale of row i of a group from what `issue` fetched (int4 with bf16 scales: the half that the index names)
        // (nvfp4: the two scale bytes in the low half of the result's bits)
        auto scale_of = [&](float raw, int gi, int i) -> float {
            if (F8 || NF || (!NV && s32)) return raw;
            const int n = weight_row(row0 + (gi * RB + i < nrows ? gi * RB + i : nrows - 1));
            const uint32_t u = __float_as_uint(raw);
            if (NV) return __uint_as_float(u >> (8 * (int)((((int64_t)n * g.K + kbase) >> 4) & 2)));
            const int64_t si = ((int64_t)n * g.K + kbase) >> g.gshift;
            return __uint_as_float((si & 1) ? u & 0xffff0000u : u << 16);
        };
        const float gsc = NV ? g.global_scale[0] : 1.0f;
        // ---- the groups of this wave's set: the next one's loads go out, then the current one is decoded and multiplied,
        // summed over the wave's lanes (fixed order: within 16 lanes by lane-permuting adds, then the four 16s in order)
        // and left in LDS for the finish
        u32x4 xv[EPL / 8];
        auto work_rows = [&](auto whole, const u32x4 (&w)[RB], const float (&sc)[RB], int gi) {
            float a[RB];
#pragma unroll
            for (int i = 0; i < RB; ++i) {
                a[i] = 0.0f;
                if (!decltype(whole)::value && gi * RB + i >= nrows) continue;     // (wave-uniform: a short last group)
                const float sv = scale_of(sc[i], gi, i);
#pragma unroll
                for (int c = 0; c < EPL / 8; ++c) {
                    u32x4 wp;
                    if constexpr (F8) wp = __builtin_bit_cast(u32x4, decode8<FMT>(w[i][2 * c], w[i][2 * c + 1], sv, 0.0f));
                    else if constexpr (NF) wp = __builtin_bit_cast(u32x4, decode8<FMT>(w[i][c], 0u, sv, 0.0f, nf4_tab[wave]));
                    else if constexpr (NV)
                        wp = __builtin_bit_cast(u32x4, decode8<FMT>(w[i][c], 0u, e4m3_to_f32((uint8_t)(__float_as_uint(sv) >> (8 * (c >> 1)))) * gsc, 0.0f));
                    else wp = __builtin_bit_cast(u32x4, decode8<FMT>(w[i][c], 0u, sv, -8.0f * sv));
#pragma unroll
                    for (int e = 0; e < 4; ++e) dot2_bf16(a[i], wp[e], xv[c][e]);
                }
                // (a dot instruction's result may be read, or its register written, by another kind of instruction only
                // 3 - 4 cycles later; the compiler keeps that distance for its own instructions and cannot see into
                // the asm above: the wait is tied to the sum, so that whatever uses it comes behind)
                asm volatile("s_nop 3" : "+v"(a[i]));
            }
            // the four rows' sums over 16 lanes each, all four at once: neighbours swap the rows they do not keep (lane l keeps
            // row l & 1 of rows 0 | 1 and of rows 2 | 3), the quad's halves likewise (lane l ends with row l & 3 summed over its
            // quad), then the four quads of the 16 lanes by two rotations and the four 16-lane rows by two swaps -- a fixed order,
            // 7 adds instead of 4 x 7
            static_assert(RB == 4, "the lanes' row exchange is written for groups of four rows");
            const bool o1 = (lane & 1) != 0, o2 = (lane & 2) != 0;
            float k01 = o1 ? a[1] : a[0], s01 = o1 ? a[0] : a[1];
            float k23 = o1 ? a[3] : a[2], s23 = o1 ? a[2] : a[3];
            k01 += lane_perm<0xB1>(s01);
            k23 += lane_perm<0xB1>(s23);
            float kk = o2 ? k23 : k01;
            const float ss = o2 ? k01 : k23;
            kk += lane_perm<0x4E>(ss);
            kk += lane_perm<0x124>(kk);               // the quad four lanes on (rotation within 16 lanes)
            kk += lane_perm<0x128>(kk);               // and the pair of quads eight lanes on
            kk = sum_rows_of_16(kk);
            if (lane < 4) red[st * g.gmax + gi][lane][ws] = kk;
        };
        auto work = [&](const u32x4 (&w)[RB], const float (&sc)[RB], int gi) {
            if (gi * RB + RB <= nrows) work_rows(std::true_type{}, w, sc, gi);
            else work_rows(std::false_type{}, w, sc, gi);
        };
        if (gcount > 0) {
            u32x4 wa[RB], wb[RB];
            float sa[RB], sb[RB];
            issue(wa, sa, 0);
#pragma unroll
            for (int c = 0; c < EPL / 8; ++c) xv[c] = *(const u32x4*)(g.x + kbase + 8 * c);
            // (the steps are written out by the state of the two buffers, so that no step waits for more than its own loads)
            int gi = 0;
            while (gi + 2 < gcount) {
                issue(wb, sb, gi + 1);
                work(wa, sa, gi);
                issue(wa, sa, gi + 2);
                work(wb, sb, gi + 1);
                gi += 2;
            }
            if (gi + 1 < gcount) {
                issue(wb, sb, gi + 1);
                work(wa, sa, gi);
                work(wb, sb, gi + 1);
            } else {
                work(wa, sa, gi);
            }
        }
        __syncthreads();
        return;
    }

    // ---- the last wave.  First the slot's launch count (its block's copy) and the B rows and bias of the rows it will
    // finish: lane t finishes row t % RB of the block's group slot t / RB = set * gmax + group of the set.  The block is
    // counted in once the count has been read.
    const int f_slot = lane / RB, f_i = lane - f_slot * RB;
    const int f_set = f_slot / g.gmax, f_gi = f_slot - f_set * g.gmax;
    const int f_row = f_gi * RB + f_i;                // row within the set's range
    const int fj = (bx * g.sets + f_set) * g.rps + f_row;          // row of the walk
    const bool finisher = f_set < g.sets && f_row < g.rps && fj < g.N;
    const int fn = weight_row(finisher ? fj : 0);     // row of the weight
    uint32_t gen = 0;
    f32x4 brow[4];
    float bias_v = 0.0f;
    if (lora) {
        // (past the caches: it is not needed before the first look at the parts has returned)
        gen = __hip_atomic_load(g.slot + kSlotCtl + (blk % kCtlCopies) * kCtlStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        brow[q] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        if (finisher && lora && 4 * q < g.r) brow[q] = *(const f32x4*)(g.lora_B + (int64_t)fn * g.r + 4 * q);
    }
    if (finisher && g.bias) bias_v = bf16_to_f32(g.bias[fn]);
    if (lora && lane == 0) {
        uint32_t one = 1u;
        asm volatile("" : "+v"(one) : "v"(gen));       // (the add may not move ahead of the point where `gen` is in its register)
        __hip_atomic_fetch_add(g.slot + kSlotCtl + (kCtlCopies + blk % kCtlCopies) * kCtlStride, one, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
    }
    // ---- while the sets stream: collect all parts -- lane (q, j) takes rank j of the parts q, q + 4, ... -- looking past
    // the caches until they carry this launch's tag
    float zv = 0.0f;                                  // lane j < 16 (and the lanes 16 apart): z[j] * scaling
    bool whole = true;
    if (lora) {
        const bool closer = blk == nb - 1;
        const bool failed_slot = gen == kGenPoison;
        bool missing = failed_slot, open = closer && !failed_slot;
        float z = 0.0f;
        int spins = 0;
        if (!failed_slot) for (;;) {
            uint64_t zt[kSuMaxParts / 4];
#pragma unroll
            for (int u = 0; u < kSuMaxParts / 4; ++u) {
                const int p = 4 * u + (lane >> 4);
                zt[u] = 0;
                if (4 * u < g.nsu)
                    zt[u] = __hip_atomic_load((const uint64_t*)g.slot + (p < g.nsu ? p : g.nsu - 1) * 256 + (lane & 15), __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
            }
            uint32_t started = 0;
            if (open && lane < kCtlCopies)
                started = __hip_atomic_load(g.slot + kSlotCtl + (kCtlCopies + lane) * kCtlStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            z = 0.0f;
            missing = false;
#pragma unroll
            for (int u = 0; u < kSuMaxParts / 4; ++u) {
                const bool have = 4 * u + (lane >> 4) < g.nsu;
                missing |= have && (uint32_t)(zt[u] >> 32) != gen + 1;
                z += have ? __uint_as_float((uint32_t)zt[u]) : 0.0f;
            }
            missing = __any(missing);
            if (open) {
#pragma unroll
                for (int d = 32; d >= 1; d >>= 1) started += __shfl_xor(started, d, 64);
                if (started == (uint32_t)nb) {
                    if (lane < kCtlCopies) {
                        __hip_atomic_store(g.slot + kSlotCtl + lane * kCtlStride, gen + 1 == kGenPoison ? 0u : gen + 1, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
                        __hip_atomic_store(g.slot + kSlotCtl + (kCtlCopies + lane) * kCtlStride, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    }
                    open = false;
                }
            }
            if (!(missing || open) || ++spins >= g.spin_limit) break;
            __builtin_amdgcn_s_sleep(8);
        }
        // (a closer that gave up marks the slot failed; a block that is about to write NaN says so: as in the kernel above)
        if (open && lane < kCtlCopies)
            __hip_atomic_store(g.slot + kSlotCtl + lane * kCtlStride, kGenPoison, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if ((missing || open) && lane == 0) __hip_atomic_fetch_add(g.fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        z += __shfl_xor(z, 16, 64);                   // the four lanes of a rank: (q0 + q1) + (q2 + q3)
        z += __shfl_xor(z, 32, 64);
        zv = (lane & 15) < g.r ? z * g.su_scale : 0.0f;
        whole = !(missing || open);
    }
    __syncthreads();

    // ---- outputs: the waves' sums in wave order, the low-rank term rank by rank, the bias
    float o = 0.0f;
    if (finisher)
        for (int ww = 0; ww < g.nw; ++ww) o += red[f_slot][f_i][ww];
    if (lora) {
#pragma unroll
        for (int j = 0; j < 16; ++j) o = __builtin_fmaf(read_lane(zv, j), brow[j >> 2][j & 3], o);
        if (!whole) o = __builtin_nanf("");
    }
    if (g.bias) o += bias_v;
    if constexpr (GU) {
        // (RB and the sets' ranges are even: lane t even holds a column's gate, lane t + 1 its up)
        const float up = lane_perm<0xB1>(o);
        const float gate = round_bf16(o);
        if (finisher && !(lane & 1)) g.y[fj >> 1] = to_bf16(round_bf16(gate * sigmoid_f32(gate)) * round_bf16(up));
    } else {
        if (finisher) g.y[fn] = to_bf16(o);
    }
}

template <int FMT, int RB, bool GU>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(FMT == XQ_FMT_FP8 ? 6 : 5, 8))) skinny_gemv_kernel(GemvArgs g) {
    skinny_gemv_body<FMT, RB, GU>(g, (int)blockIdx.x, (int)gridDim.x);
}

// several forwards on one x (same format and K, hence the same block shape) in one grid: first the blocks that form the
// parts of z, forward by forward (so that none of them waits behind another forward's rows for a CU), then the streaming
// blocks, forward by forward; a block finds its forward by its index (the boundaries are leading scalars, with the wave
// from the start).  p1 .. p4, s1 .. s4: blocks of either kind before the second, third, fourth forward and in all.
struct GemvBatch {
    GemvArgs job[kRowsMaxJobs];
};
template <int FMT, int RB>
__global__ void __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(FMT == XQ_FMT_FP8 ? 6 : 5, 8)))
skinny_gemv_multi_kernel(int32_t p1, int32_t p2, int32_t p3, int32_t p4, int32_t s1, int32_t s2, int32_t s3, int32_t s4, GemvBatch b) {
    const int bx = (int)blockIdx.x;
    const bool forms_z = bx < p4;
    const int c = forms_z ? bx : bx - p4;             // index among the blocks of its kind
    const int f1 = forms_z ? p1 : s1, f2 = forms_z ? p2 : s2, f3 = forms_z ? p3 : s3;
    const int i = (c >= f1 ? 1 : 0) + (c >= f2 ? 1 : 0) + (c >= f3 ? 1 : 0);   // uniform
    const int plo = i == 0 ? 0 : i == 1 ? p1 : i == 2 ? p2 : p3, phi = i == 0 ? p1 : i == 1 ? p2 : i == 2 ? p3 : p4;
    const int slo = i == 0 ? 0 : i == 1 ? s1 : i == 2 ? s2 : s3, shi = i == 0 ? s1 : i == 1 ? s2 : i == 2 ? s3 : s4;
    const int nsu = phi - plo;                        // this forward's blocks that form z come first in its own count
    skinny_gemv_body<FMT, RB, false>(b.job[i], forms_z ? c - plo : nsu + (c - slo), nsu + (shi - slo));
}

static std::atomic<int> g_skinny_gemv{[] { const char* e = getenv("XQ_SKINNY_GEMV"); return e ? atoi(e) : 1; }()};
void set_skinny_gemv(int on) { g_skinny_gemv = on != 0; }

// a launch's shape: sets of K / 1024 waves, as many to a block as make up to 8 streaming waves; as many blocks as the CUs
// hold at once (20 of a CU's 24 waves: two blocks of 9 waves, one of 13; the rest is room for the blocks that form z)
// where the weight has that many groups of rows, more blocks where a block's sets would otherwise get more than
// kGemvSlots groups
struct GemvPlan {
    int nw, sets, gmax, rps;
    unsigned blocks;
};
// `share`: this forward's part of the blocks that the CUs hold at once (1 for a launch of its own; in a joint launch the
// forwards split them by their rows).  `even`: ranges of an even number of rows (gate | up walked in pairs).
static GemvPlan gemv_plan(const xq_weight* w, double share = 1.0, bool even = false) {
    GemvPlan p;
    p.nw = (int)((w->format == XQ_FMT_FP8 ? w->cols : w->cols / 2) / 1024);
    p.sets = 8 / p.nw > 1 ? 8 / p.nw : 1;
    const int cap = (kGemvSlots / p.sets) * kGemvRows;     // rows of a set at most
    // blocks: what the CUs hold at once at most (two blocks of 9 waves each, one of 13), fewer where the sets would get
    // less than two groups of rows each (a block that lasts two steps hides its wait for the low-rank parts behind the
    // second; measured on block-fp8 [4096, 4096]: 7.0 us against 8.3 with one step per set; int4, whose time is its
    // decode, wants all the blocks it can have) but not fewer than one per CU, nor more than there are groups
    const int per_cu = 20 / (p.sets * p.nw + 1) > 1 ? 20 / (p.sets * p.nw + 1) : 1;
    int64_t fill = (int64_t)(256 * per_cu * share + 0.5), floor_ = (int64_t)(256 * share + 0.5);
    if (fill < 1) fill = 1;
    if (floor_ < 1) floor_ = 1;
    const int64_t two_steps = xq_cdiv(w->rows, (int64_t)p.sets * 2 * kGemvRows);
    int64_t nb = w->format != XQ_FMT_FP8 ? fill : two_steps > floor_ ? two_steps : floor_;
    if (nb > fill) nb = fill;
    if (nb > xq_cdiv(w->rows, (int64_t)p.sets * kGemvRows)) nb = xq_cdiv(w->rows, (int64_t)p.sets * kGemvRows);
    if (xq_cdiv(w->rows, (int64_t)p.sets * cap) > nb) nb = xq_cdiv(w->rows, (int64_t)p.sets * cap);
    p.blocks = (unsigned)nb;
    p.rps = (int)xq_cdiv(w->rows, nb * p.sets);            // the rows dealt evenly: a set's range is at most one row longer than another's
    if (even) p.rps += p.rps & 1;                          // (cap is even)
    p.gmax = (int)xq_cdiv(p.rps, kGemvRows);
    return p;
}

bool skinny_gemv_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r) {
    if (!g_skinny_gemv || M != 1 || w->num_experts != 1 || w->layout != XQ_LAYOUT_FLAT) return false;
    if (w->format == XQ_FMT_FP8) {
        if (w->scale_dtype != XQ_SCALE_F32) return false;
    } else if (w->format == XQ_FMT_NF4) {
        if (w->scale_dtype != XQ_SCALE_F32 || w->group != 64) return false;
    } else if (w->format == XQ_FMT_NVFP4) {
        if (w->scale_dtype != XQ_SCALE_E4M3 || w->group != 16 || !w->global_scale) return false;
    } else if (w->format != XQ_FMT_INT4 || w->group < 32 || (w->group & (w->group - 1)) != 0 ||
               (w->scale_dtype != XQ_SCALE_F32 && w->scale_dtype != XQ_SCALE_BF16)) {
        return false;
    }
    // (bf16 scales are read as the aligned words that hold them: the array must end on a word)
    if (w->format == XQ_FMT_INT4 && (w->rows * w->cols / w->group) % 2 != 0) return false;
    // int4 is decode-bound in either kernel; this one is ahead where the other's organisation fits badly -- few rows (q, kv)
    // or long ones (down: -15 %) -- and 3 % behind on many short rows (gate/up [12288, 4096], [24576, 4096]), which stay there
    if (w->format == XQ_FMT_INT4 && w->rows > 4096 && w->cols < 8192) return false;
    const int64_t row_bytes = w->format == XQ_FMT_FP8 ? w->cols : w->cols / 2;
    if (row_bytes % 1024 != 0 || row_bytes / 1024 > 15 || w->rows < 1 || w->rows >= (1ll << 30)) return false;
    if (!xq_aligned(w->packed, 16)) return false;
    if (r > 0) {
        if (lora_dtype != XQ_DT_F32 || r > 16 || r % 4 != 0 || !xq_aligned(lora_A, 16) || !xq_aligned(lora_B, 16)) return false;
        if (w->cols % kSuPartK != 0 || w->cols / kSuPartK > kSuMaxParts) return false;
    }
    return true;
}

static int gemv_args(const xq_weight* w, const GemvPlan& p, const bf16_t* x, const void* lora_A, const void* lora_B, int r, float scaling,
                     const bf16_t* bias, bf16_t* y, const void* slot_key, hipStream_t stream, GemvArgs* out) {
    XQ_REQUIRE(p.sets * p.gmax <= kGemvSlots && p.sets * p.nw >= 4 && (p.sets * p.nw + 1) * 64 <= 1024,
               "xq_linear_fwd: internal error: dot-product launch out of range");
    GemvArgs& g = *out;
    g.x = x; g.N = (int)w->rows; g.K = (int)w->cols;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.gshift = 0;
    for (int v = w->group; v > 1; v >>= 1) ++g.gshift;
    g.scale_dtype = w->scale_dtype;
    g.lora_A = (const float*)lora_A; g.lora_B = (const float*)lora_B; g.r = r; g.su_scale = scaling;
    g.bias = bias; g.y = y;
    g.nsu = r > 0 ? (int)(w->cols / kSuPartK) : 0;
    g.nw = p.nw; g.sets = p.sets; g.gmax = p.gmax; g.rps = p.rps;
    g.slot = nullptr; g.fail = nullptr;
    g.spin_limit = g_rows_spin_limit.load();
    if (r > 0) return rows_slot(slot_key, stream, &g.slot, &g.fail);
    return XQ_OK;
}

// swiglu: w is gate | up [2 I, K] and y is h [I]
int launch_skinny_gemv(const xq_weight* w, const bf16_t* x, const void* lora_A, const void* lora_B, int r, float scaling,
                       const bf16_t* bias, bf16_t* y, const void* slot_key, hipStream_t stream, bool swiglu) {
    const GemvPlan p = gemv_plan(w, 1.0, swiglu);
    GemvArgs g;
    const int rc = gemv_args(w, p, x, lora_A, lora_B, r, scaling, bias, y, slot_key, stream, &g);
    if (rc) return rc;
    const unsigned grid = p.blocks + (unsigned)g.nsu, threads = (unsigned)((p.sets * p.nw + 1) * 64);
    if (w->format == XQ_FMT_FP8) {
        if (swiglu) skinny_gemv_kernel<XQ_FMT_FP8, kGemvRows, true><<<grid, threads, 0, stream>>>(g);
        else skinny_gemv_kernel<XQ_FMT_FP8, kGemvRows, false><<<grid, threads, 0, stream>>>(g);
    } else if (w->format == XQ_FMT_NF4) {
        if (swiglu) skinny_gemv_kernel<XQ_FMT_NF4, kGemvRows, true><<<grid, threads, 0, stream>>>(g);
        else skinny_gemv_kernel<XQ_FMT_NF4, kGemvRows, false><<<grid, threads, 0, stream>>>(g);
    } else if (w->format == XQ_FMT_NVFP4) {
        if (swiglu) skinny_gemv_kernel<XQ_FMT_NVFP4, kGemvRows, true><<<grid, threads, 0, stream>>>(g);
        else skinny_gemv_kernel<XQ_FMT_NVFP4, kGemvRows, false><<<grid, threads, 0, stream>>>(g);
    } else {
        if (swiglu) skinny_gemv_kernel<XQ_FMT_INT4, kGemvRows, true><<<grid, threads, 0, stream>>>(g);
        else skinny_gemv_kernel<XQ_FMT_INT4, kGemvRows, false><<<grid, threads, 0, stream>>>(g);
    }
    return XQ_OK;
}

// several forwards (same format and K) in one grid; each has its own slot, keyed 256 bytes apart inside the caller's workspace
static int launch_skinny_gemv_multi(const SkinnyRowsJob* jobs, int n_jobs, const bf16_t* x, const void* slot_key, hipStream_t stream) {
    int64_t rows = 0;
    for (int i = 0; i < n_jobs; ++i) rows += jobs[i].w->rows;
    GemvBatch b;
    int32_t pf[kRowsMaxJobs + 1], sf[kRowsMaxJobs + 1];   // blocks that form z / that stream, before each forward
    int pat = 0, sat = 0;
    unsigned threads = 0;
    for (int i = 0; i < kRowsMaxJobs; ++i) {
        pf[i] = pat;
        sf[i] = sat;
        if (i >= n_jobs) {
            b.job[i] = b.job[0];
            continue;
        }
        const GemvPlan p = gemv_plan(jobs[i].w, (double)jobs[i].w->rows / (double)rows);
        const int rc = gemv_args(jobs[i].w, p, x, jobs[i].lora_A, jobs[i].lora_B, jobs[i].r, jobs[i].scaling, jobs[i].bias, jobs[i].y,
                                 (const char*)slot_key + 256 * i, stream, &b.job[i]);
        if (rc) return rc;
        pat += b.job[i].nsu;
        sat += (int)p.blocks;
        threads = (unsigned)((p.sets * p.nw + 1) * 64);
    }
    pf[kRowsMaxJobs] = pat;
    sf[kRowsMaxJobs] = sat;
    const unsigned grid = (unsigned)(pat + sat);
    if (jobs[0].w->format == XQ_FMT_FP8)
        skinny_gemv_multi_kernel<XQ_FMT_FP8, kGemvRows><<<grid, threads, 0, stream>>>(pf[1], pf[2], pf[3], pf[4], sf[1], sf[2], sf[3], sf[4], b);
    else if (jobs[0].w->format == XQ_FMT_NF4)
        skinny_gemv_multi_kernel<XQ_FMT_NF4, kGemvRows><<<grid, threads, 0, stream>>>(pf[1], pf[2], pf[3], pf[4], sf[1], sf[2], sf[3], sf[4], b);
    else if (jobs[0].w->format == XQ_FMT_NVFP4)
        skinny_gemv_multi_kernel<XQ_FMT_NVFP4, kGemvRows><<<grid, threads, 0, stream>>>(pf[1], pf[2], pf[3], pf[4], sf[1], sf[2], sf[3], sf[4], b);
    else
        skinny_gemv_multi_kernel<XQ_FMT_INT4, kGemvRows><<<grid, threads, 0, stream>>>(pf[1], pf[2], pf[3], pf[4], sf[1], sf[2], sf[3], sf[4], b);
    return XQ_OK;
}

// ---- gate | up with the SwiGLU finish: h = silu(gate) * up from one weight [2 I, K] in one launch
template <int FMT, int NJ, int MR>
static int launch_rows_gu_one(const SkinnyRowsArgs& g, unsigned grid, size_t lds, hipStream_t s) {
    static std::atomic<bool> attr_set{false};
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)skinny_rows_kernel_p<FMT, 3, NJ, MR, 2, true>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) {
            xq_set_error("xq_linear_fwd_swiglu: cannot raise the dynamic LDS limit: %s", hipGetErrorString(e));
            return XQ_ERR_LAUNCH;
        }
        attr_set = true;
    }
    skinny_rows_kernel_p<FMT, 3, NJ, MR, 2, true><<<grid, 512, lds, s>>>(g.x, (int32_t)g.ldx, g.M, g.N, g.K, g.packed, g.scales, g.slot, g.lora_A, g.nsu,
                                                                          g.gshift | g.scale_dtype << 8, g);
    return XQ_OK;
}

template <int FMT, int NJ>
static int launch_rows_gu_mr(const SkinnyRowsArgs& g, int MR, unsigned grid, size_t lds, hipStream_t s) {
    if (MR == 1) return launch_rows_gu_one<FMT, NJ, 1>(g, grid, lds, s);
    if (MR == 8) return launch_rows_gu_one<FMT, NJ, 8>(g, grid, lds, s);
    return launch_rows_gu_one<FMT, NJ, 16>(g, grid, lds, s);
}

// true when w [2 I, K] takes the one-launch kernel in two rounds of three row groups, so that a block can hold the gate and
// the up rows of the same 48 columns
bool skinny_rows_swiglu_supported(const xq_weight* w, int64_t M, const void* lora_A, const void* lora_B, int lora_dtype, int r) {
    if (w->rows % 2 != 0 || !skinny_rows_supported(w, M, lora_A, lora_B, lora_dtype, r)) return false;
    RowsPlan p;
    if (!rows_plan(w, M, &p)) return false;
    return p.R == 2 && p.G == 3 && (w->rows / 2) % 48 == 0 && (w->format == XQ_FMT_FP8 ? p.njt <= 8 : p.njt <= 4);
}

int launch_skinny_rows_swiglu(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B, int r,
                              float scaling, const bf16_t* bias, bf16_t* h, int64_t ldh, const void* slot_key, hipStream_t stream) {
    if (w->rows % 2 == 0 && skinny_gemv_supported(w, M, lora_A, lora_B, XQ_DT_F32, r))
        return launch_skinny_gemv(w, x, lora_A, lora_B, r, scaling, bias, h, slot_key, stream, true);
    RowsPlan p;
    XQ_REQUIRE(rows_plan(w, M, &p) && p.R == 2 && p.G == 3 && ldx < (1ll << 31),
               "xq_linear_fwd_swiglu: internal error: shape not supported by the one-launch skinny kernel");
    SkinnyRowsArgs g;
    const int rc = rows_args(w, p, x, ldx, M, lora_A, lora_B, r, scaling, bias, h, ldh, slot_key, stream, &g);
    if (rc) return rc;
    const unsigned grid = (unsigned)(w->rows / 2 / 48);
#define XQ_GU_CASE(F, NN) \
    if (w->format == F && p.njt == NN) return launch_rows_gu_mr<F, NN>(g, p.MR, grid, p.lds, stream)
    XQ_GU_CASE(XQ_FMT_FP8, 4); XQ_GU_CASE(XQ_FMT_FP8, 8);
    XQ_GU_CASE(XQ_FMT_INT4, 4); XQ_GU_CASE(XQ_FMT_NF4, 4); XQ_GU_CASE(XQ_FMT_NVFP4, 4);
#undef XQ_GU_CASE
    XQ_REQUIRE(false, "xq_linear_fwd_swiglu: internal error: no kernel for %d load steps", p.njt);
}

// ---- several forwards that share x as one launch
bool skinny_rows_multi_supported(const SkinnyRowsJob* jobs, int n_jobs, int64_t M, int lora_dtype) {
    if (n_jobs < 2 || n_jobs > kRowsMaxJobs) return false;
    const xq_weight* ws[kRowsMaxJobs];
    for (int i = 0; i < n_jobs; ++i) {
        const xq_weight* w = jobs[i].w;
        ws[i] = w;
        if (w->format != jobs[0].w->format || w->cols != jobs[0].w->cols || w->group != jobs[0].w->group ||
            w->scale_dtype != jobs[0].w->scale_dtype || w->layout != jobs[0].w->layout)
            return false;
        if (!skinny_rows_supported(w, M, jobs[i].lora_A, jobs[i].lora_B, lora_dtype, jobs[i].r)) return false;
    }
    RowsPlan p;
    if (!rows_plan_multi(ws, n_jobs, M, &p)) return false;
    for (int i = 0; i < n_jobs; ++i)
        if (jobs[i].r > 0 && ws[i]->cols / kSuPartK > xq_cdiv(ws[i]->rows / 16, p.G * p.R)) return false;   // a block forms at most one su part
    return true;
}

int launch_skinny_rows_multi(const SkinnyRowsJob* jobs, int n_jobs, const bf16_t* x, int64_t ldx, int64_t M, const void* slot_key,
                             hipStream_t stream) {
    const xq_weight* ws[kRowsMaxJobs];
    for (int i = 0; i < n_jobs; ++i) ws[i] = jobs[i].w;
    bool dots = true;                                  // one row, every forward on the dot-product kernel
    for (int i = 0; i < n_jobs; ++i) dots = dots && skinny_gemv_supported(ws[i], M, jobs[i].lora_A, jobs[i].lora_B, XQ_DT_F32, jobs[i].r);
    if (dots) return launch_skinny_gemv_multi(jobs, n_jobs, x, slot_key, stream);
    RowsPlan p;
    XQ_REQUIRE(rows_plan_multi(ws, n_jobs, M, &p), "xq_linear_fwd_multi: internal error: shapes not supported by the one-launch skinny kernel");
    SkinnyRowsBatch b;
    int first = 0;
    for (int i = 0; i < kRowsMaxJobs; ++i) {
        b.first[i] = first;
        if (i >= n_jobs) {
            b.job[i] = b.job[0];
            continue;
        }
        // each forward has a slot of its own: its key is a distinct address inside the caller's workspace
        const int rc = rows_args(ws[i], p, x, ldx, M, jobs[i].lora_A, jobs[i].lora_B, jobs[i].r, jobs[i].scaling, jobs[i].bias, jobs[i].y,
                                 jobs[i].ldy, (const char*)slot_key + 256 * i, stream, &b.job[i]);
        if (rc) return rc;
        first += (int)xq_cdiv(ws[i]->rows / 16, p.G * p.R);
    }
    b.first[kRowsMaxJobs] = first;
    switch (ws[0]->format) {
        case XQ_FMT_FP8: return launch_rows_fmt<XQ_FMT_FP8>(b.job[0], &b, p, (unsigned)first, stream);
        case XQ_FMT_INT4: return launch_rows_fmt<XQ_FMT_INT4>(b.job[0], &b, p, (unsigned)first, stream);
        case XQ_FMT_NF4: return launch_rows_fmt<XQ_FMT_NF4>(b.job[0], &b, p, (unsigned)first, stream);
        default: return launch_rows_fmt<XQ_FMT_NVFP4>(b.job[0], &b, p, (unsigned)first, stream);
    }
}

}  // namespace xq
