// Skinny-M (M <= 64) fused dequant-GEMM forward: the HBM-bound decode/rollout regime.
//
//   y[M, N] = x[M, K] . deq(W)^T + bias + s * (x . A^T) . B^T          (W FLAT [N, K])
//
// Every byte of the packed weight is read from HBM exactly once, decoded in registers to the exact bf16
// value of the reference decoder and fed to v_mfma_f32_32x32x16_bf16 against x fragments.  Two launches per
// forward, no atomics, no zeroed buffers, fixed summation orders (deterministic):
//
//  1. skinny_split_kernel: a grid of (128-row block) x (K split) tiles.  A block's four waves own 32 weight
//     rows each and the same K range of at most four 128-element chunks.  Every load is unconditional and
//     issued ahead of its use with exactly counted waits: the x slice first, then the weight chunks as a
//     stream with two chunks in flight (a chunk's registers are requested again once it has been multiplied),
//     and the number of K splits is chosen so that the whole grid is resident at once (four blocks per CU at
//     M <= 16, three above).  Weight loads are coalesced (a load instruction covers whole rows of a chunk) and
//     reach the MFMA layout through a wave-private XOR-swizzled LDS slab; x goes through LDS once per block
//     and is shared by the four waves: the whole [rows, K range] slice up to 32 rows, chunk by chunk (all 64
//     rows of 128 elements, two buffers) above, so that a weight chunk is decoded once whatever M is.  Each
//     block stores its fp32 partial tile to part[split][M][N]; the first row of blocks carries no weight rows
//     and computes the low-rank intermediate su = x . A^T for one K split each.
//  2. skinny_epilogue_kernel: sums the splits in order, adds bias and s * su . B^T in fp32 and rounds once
//     to bf16.
//
// Measured per forward on an MI355X, launches back to back (block_fp8, r = 16): 4096->12288 (48 MiB) 15.6 us
// at M = 1, 21 us at M = 32, 31 us at M = 64; 4096->1024 (4 MiB) 8 us at M = 1.  A kernel that only reads
// the 48 MiB takes 8-9 us.  (M <= 16 normally takes the one-launch kernel of xq_skinny_rows.hip instead.)
#include <stdlib.h>

#include "xq_common.h"
#include "xq_lora.h"
#include "xq_skinny.h"

namespace xq {

struct SkinnyArgs {
    const bf16_t* x;
    int64_t ldx;
    int32_t M, N, K;
    const uint8_t* packed;
    const uint8_t* scales;
    const float* global_scale;
    int32_t group, scale_dtype;
    int32_t splits;            // K splits
    int32_t su_blocks;         // leading grid rows (0 or 1) whose blocks compute the su part of their split
    int32_t chunk_q, chunk_rem; // 128-element chunks per split: chunk_q, one more in the first chunk_rem splits
    int32_t xp;                // LDS row pitch of the x slice in bf16 elements (longest split + 8)
    float* partial;            // [splits][M][N]
    float* su_part;            // [splits * 4][M][r_pad]
    const void* lora_A;        // [r, K] fp32 or bf16
    int32_t lora_f32, r, r_pad;
};

struct SkinnyEpiArgs {
    const float* partial;
    const float* su_part;
    int32_t splits, su_parts, M, N;
    const void* lora_B;        // [N, r] fp32 or bf16
    int32_t lora_f32, r, r_pad;
    float su_scale;
    const bf16_t* bias;
    bf16_t* y;
    int64_t ldy;
};

// One block = 128 weight rows x one K split (or, for the leading su blocks, the x . A^T part of one split).
// MR = 16, 32 or 64 bounds M.  Up to 32 rows the split's whole x slice is staged in LDS once; at MR = 64 weight
// blocks take x one 128-element chunk at a time (all 64 rows, two LDS buffers), so that a weight chunk is decoded
// once and multiplied into both halves of the rows, and three blocks still fit a CU.  (The su blocks at MR = 64
// stage their x rows 32 at a time.)
// The arguments that the first loads need are the leading scalars: the hardware hands a kernel's first 14 argument dwords
// to each wave in registers (where the platform supports it; otherwise they are fetched like the rest), so those loads do
// not wait for a round trip to the argument block.  fmt_bits = group | scale_dtype << 24, split_bits = splits |
// su_blocks << 16, chunk_bits = chunk_q | chunk_rem << 16; `rest` carries the other fields (its copies of these are unused).
template <int FMT, int MR, int NCH>
__global__ void __launch_bounds__(256, MR == 16 ? 4 : 3)
skinny_split_kernel(const bf16_t* x_, int32_t ldx_, int32_t M_, int32_t N_, int32_t K_, const uint8_t* packed_, const uint8_t* scales_,
                    int32_t fmt_bits, int32_t split_bits, int32_t chunk_bits, int32_t xp_, SkinnyArgs rest) {
    constexpr int TR = MR < 32 ? MR : 32;              // x rows staged at a time
    constexpr int NPASS = MR / TR;
    SkinnyArgs g = rest;
    g.x = x_; g.ldx = ldx_; g.M = M_; g.N = N_; g.K = K_; g.packed = packed_; g.scales = scales_;
    g.group = fmt_bits & 0xFFFFFF; g.scale_dtype = fmt_bits >> 24;
    g.splits = split_bits & 0xFFFF; g.su_blocks = split_bits >> 16;
    g.chunk_q = chunk_bits & 0xFFFF; g.chunk_rem = chunk_bits >> 16;
    g.xp = xp_;
    // The other arguments are pinned in scalar registers in one go once the first loads are out (left to the compiler,
    // argument loads are placed lazily, each batch with its own wait).
    auto pin_rest = [&]() {
        asm volatile("" ::"s"(g.global_scale), "s"(g.partial), "s"(g.su_part), "s"(g.lora_A), "s"(g.lora_f32), "s"(g.r), "s"(g.r_pad));
    };
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    bf16_t* xs = (bf16_t*)smem;                                  // [min(M, 32) rows][xp]; fragment rows past M read row 0:
    const int XP = g.xp;                                         // they feed only output columns >= M, which are never stored
    const int xrows = g.M < 32 ? g.M : 32;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int fr = lane & 31, fh = lane >> 5;
    constexpr int EB = FMT == XQ_FMT_FP8 ? 1 : 2;      // elements per byte
    constexpr int NLOAD = FMT == XQ_FMT_FP8 ? 4 : 2;   // 16-byte loads per lane per 128-k chunk
    constexpr int NSC = FMT == XQ_FMT_NVFP4 ? 4 : FMT == XQ_FMT_NF4 ? 2 : 1;   // scale registers per chunk

    // grid: x = K split, y = 128-row block, preceded by one row of su blocks when there is a low-rank term
    const int split = blockIdx.x;
    const bool su_block = (int)blockIdx.y < g.su_blocks;
    const int rb = su_block ? 0 : (int)blockIdx.y - g.su_blocks;
    // the first `chunk_rem` splits hold chunk_q + 1 chunks of 128 elements, the others chunk_q (no divisions here:
    // nothing is in flight until the loads below are issued)
    const int c_begin = split * g.chunk_q + (split < g.chunk_rem ? split : g.chunk_rem);
    const int nch = g.chunk_q + (split < g.chunk_rem ? 1 : 0);   // 1 .. NCH (the launcher guarantees it)
    const int c_end = c_begin + nch;
    const int k_begin = c_begin << 7;

    // ---- x slice [rows of pass h][nch*128]: coalesced 16-byte pieces, row-major over the block's threads.  Every
    // load of this kernel is unconditional (rows and chunks past the end are clamped onto valid ones and their
    // data ignored): with no branches between the loads and their uses the waits count exactly, so the x slice
    // is staged and each weight chunk decoded while the chunks behind it are still in flight.
    // Thread t owns column piece t % (NCH*16) of rows t / (NCH*16) + i * (16/NCH); pieces past the split's own
    // nch*16 columns (a split shorter than NCH chunks) are loaded clamped and never stored.
    constexpr int XL = TR * NCH / 16;                            // pieces per thread: TR rows x NCH*16 / 256
    constexpr int CPR = NCH * 16, RSTEP = 16 / NCH;              // column pieces per row, rows per step
    const int ppr = nch << 4;                                    // pieces of a row that belong to this split
    u32x4 xr[XL];
    auto load_x = [&](int h, int t) {
        const int col = t % CPR < ppr ? t % CPR : ppr - 1;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int row = h * 32 + t / CPR + i * RSTEP;
            xr[i] = *(const u32x4*)(g.x + (int64_t)(row < g.M ? row : g.M - 1) * g.ldx + k_begin + col * 8);
        }
    };
    // block barrier on LDS traffic only: __syncthreads() would also wait for every weight load in flight
    auto lds_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    auto stage_x = [&](int h, int t) {
        const int col = t % CPR;
#pragma unroll
        for (int i = 0; i < XL; ++i) {
            const int row = t / CPR + i * RSTEP;
            if (col < ppr && h * 32 + row < g.M) *(u32x4*)(xs + row * XP + col * 8) = xr[i];
        }
        lds_barrier();
    };
    // a value the optimiser cannot see through: index arithmetic derived from it inside a loop is redone per
    // iteration instead of being hoisted into (and spilling) registers held across the whole loop
    auto opaque = [](int v) { asm volatile("" : "+v"(v)); return v; };
    if (MR < 64 || su_block) load_x(0, tid);      // (weight blocks at MR = 64 take x chunk by chunk, see below)

    if (su_block) {
        pin_rest();
        // su part of this split, D[rank][m] (ranks >= r are zero): wave w takes the k16 steps t = w, w+4, ...; the
        // four sums meet in LDS (behind the x slice) in wave order.  The factor rows are fetched with unconditional
        // 16-byte loads (rows and steps past the end clamped, their values masked), the first rank tile's together
        // with the x slice.
        const int steps = nch << 3;
        float* out = g.su_part + (int64_t)split * g.M * g.r_pad;
        float* red = (float*)(smem + (size_t)xrows * XP * 2);      // [4 waves][16 regs][64 lanes]
        u32x4 ar[2 * NCH][2];
        auto load_a = [&](int jt) {
            const int rrow = jt * 32 + fr;
            const int64_t base = (int64_t)(rrow < g.r ? rrow : 0) * g.K + k_begin + fh * 8;
#pragma unroll
            for (int u = 0; u < 2 * NCH; ++u) {
                const int t = wave + 4 * u < steps ? wave + 4 * u : steps - 1;
                if (g.lora_f32) {
                    ar[u][0] = *(const u32x4*)((const float*)g.lora_A + base + t * 16);
                    ar[u][1] = *(const u32x4*)((const float*)g.lora_A + base + t * 16 + 4);
                } else {
                    ar[u][0] = *(const u32x4*)((const bf16_t*)g.lora_A + base + t * 16);
                }
            }
        };
        load_a(0);
        for (int jt = 0; jt < ((g.r_pad + 31) >> 5); ++jt) {
            if (jt > 0) load_a(jt);
            const bool rvalid = jt * 32 + fr < g.r;
            bf16x8 af[2 * NCH];
#pragma unroll
            for (int u = 0; u < 2 * NCH; ++u) {
                u32x4 v = ar[u][0];
                if (g.lora_f32) {
                    v = u32x4{pack_bf16x2(__uint_as_float(ar[u][0][0]), __uint_as_float(ar[u][0][1])),
                              pack_bf16x2(__uint_as_float(ar[u][0][2]), __uint_as_float(ar[u][0][3])),
                              pack_bf16x2(__uint_as_float(ar[u][1][0]), __uint_as_float(ar[u][1][1])),
                              pack_bf16x2(__uint_as_float(ar[u][1][2]), __uint_as_float(ar[u][1][3]))};
                }
                if (!rvalid || wave + 4 * u >= steps) v = u32x4{0, 0, 0, 0};
                af[u] = __builtin_bit_cast(bf16x8, v);
            }
#pragma unroll 1
            for (int h = 0; h < NPASS; ++h) {
                if (h * 32 < g.M) {
                    // the x tile in LDS is current only for a single pass and the first rank tile
                    if (NPASS > 1 || jt == 0) {
                        if (h > 0 || jt > 0) load_x(h, tid);       // earlier reads of the tile are behind two barriers
                        stage_x(h, tid);
                    }
                    const int xrow = h * 32 + fr < g.M ? fr : 0;
                    f32x16 sacc;
#pragma unroll
                    for (int q = 0; q < 16; ++q) sacc[q] = 0.0f;
#pragma unroll
                    for (int u = 0; u < 2 * NCH; ++u) {
                        const int t = wave + 4 * u;
                        if (t < steps) {
                            const bf16x8 xf = *(const bf16x8*)(xs + xrow * XP + t * 16 + fh * 8);
                            sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[u], xf, sacc, 0, 0, 0);
                        }
                    }
                    __syncthreads();   // the previous sums have been read
#pragma unroll
                    for (int q = 0; q < 16; ++q) red[(wave * 16 + q) * 64 + lane] = sacc[q];
                    __syncthreads();
                    // wave w sums register quad w of every lane: ranks jt*32 + 8w + 4*fh .. +3 of row m = 32h + fr
                    f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                    for (int ww = 0; ww < 4; ++ww)
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] += red[(ww * 16 + wave * 4 + e) * 64 + lane];
                    const int j0 = jt * 32 + 8 * wave + 4 * fh, m = h * 32 + fr;
                    if (m < g.M && j0 < g.r_pad) *(f32x4*)(out + (int64_t)m * g.r_pad + j0) = v;
                }
            }
        }
        return;
    }

    // ---- the block's whole weight tile -> registers, fetched coalesced: a load instruction covers whole
    // rows of the chunk (lane l: row l / PPR of the instruction's rows, 16-byte piece l % PPR)
    constexpr int PPR = FMT == XQ_FMT_FP8 ? 8 : 4;     // 16-byte pieces per row per 128-k chunk
    constexpr int RPI = 64 / PPR;                      // rows per load instruction
    const int lrow = lane / PPR, lpiece = lane % PPR;
    const int nbase = rb * 128 + wave * 32;
    int n = nbase + fr;                                 // the row this lane feeds to the MFMA
    n = n < g.N ? n : g.N - 1;
    // A single pass over the weights (M <= 32) takes them as a short stream: two chunks in flight, a chunk's registers
    // refilled with the chunk two further on once it has been multiplied.  A CU accepts loads only as fast as memory
    // returns them, and with every chunk of its 12 to 16 waves requested at once the waves placed last start late and
    // have all their decode work left when the stream ends.  (M > 32 takes the same stream with x chunk by chunk, below.)
    constexpr int DC = NCH > 2 ? 2 : NCH;
    u32x4 w[DC][NLOAD];
    uint32_t sc[DC][NSC];
    const bool int4_small_group = FMT == XQ_FMT_INT4 && (g.group & 127) != 0;   // looked up per 8 elements at use
    const uint8_t* wp[NLOAD];
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
        int nl = nbase + RPI * i + lrow;
        nl = nl < g.N ? nl : g.N - 1;
        wp[i] = g.packed + ((int64_t)nl * g.K) / EB + lpiece * 16;
    }
    auto load_chunk = [&](int c_) {
        {
            const int c = c_ % DC;
            const int cc = c_begin + c_ < c_end ? c_begin + c_ : c_end - 1;
#pragma unroll
            for (int i = 0; i < NLOAD; ++i) w[c][i] = *(const u32x4*)(wp[i] + (int64_t)cc * (128 / EB));
            if (FMT == XQ_FMT_FP8) sc[c][0] = ((const uint32_t*)g.scales)[(n >> 7) * ((g.K + 127) >> 7) + cc];
            else if (FMT == XQ_FMT_INT4) {
                const int64_t si = int4_small_group ? 0 : ((int64_t)n * g.K + cc * 128) / g.group;
                sc[c][0] = g.scale_dtype == XQ_SCALE_F32 ? ((const uint32_t*)g.scales)[si] : ((const uint16_t*)g.scales)[si];
            } else if (FMT == XQ_FMT_NF4) {
                const u32x2 t = *(const u32x2*)((const uint32_t*)g.scales + (((int64_t)n * g.K + cc * 128) >> 6));   // fp32, group 64
                sc[c][0] = t[0];
                sc[c][1] = t[1];
            } else {
                const int64_t si = ((int64_t)n * g.K + cc * 128) >> 4;   // the 8 block scales of this row's chunk
                if (g.scale_dtype == XQ_SCALE_E4M3) {
                    const u32x2 t = *(const u32x2*)(g.scales + si);
                    sc[c][0] = t[0];
                    sc[c][1] = t[1];
                } else {
#pragma unroll
                    for (int j = 0; j < 4; ++j) sc[c][j] = ((const uint32_t*)g.scales)[si + 2 * j + fh];   // this lane's four
                }
            }
        }
    };
    // M > 32: all 64 x rows of one 128-element chunk at a time, requested just ahead of the chunk's weights (thread t: piece
    // t % 16 of rows t / 16 + 16 i), so that a chunk is decoded once and multiplied into both halves of the rows
    u32x4 xcr[4];                                           // one chunk's pieces: requested again as soon as they are in LDS
    auto load_xc = [&](int c_) {
        const int cc = c_begin + c_ < c_end ? c_begin + c_ : c_end - 1;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int row = (tid >> 4) + 16 * i;
            xcr[i] = *(const u32x4*)(g.x + (int64_t)(row < g.M ? row : g.M - 1) * g.ldx + cc * 128 + (tid & 15) * 8);
        }
    };
#pragma unroll
    for (int c = 0; c < DC; ++c) {
        if (MR == 64 && c == 0) load_xc(0);
        load_chunk(c);
    }
    pin_rest();

    // ---- decode + multiply: D[n][m] += deq(W)[n][k] x[m][k].  Each chunk's slab goes through a wave-private LDS
    // staging area (XOR-swizzled 16-byte pieces: writes and fragment reads are conflict free) to reach the
    // MFMA layout: lane (row fr, half fh) reads piece 2u+fh of its row for the k16 steps 2u and 2u+1, i.e. step
    // t = 2u+v covers k = 32u + 16*fh + 8v .. +7 of the chunk; the x fragments use the same map.  LDS operations
    // of one wave execute in order, so the slab is reused chunk after chunk without barriers.
    const float gsc = FMT == XQ_FMT_NVFP4 ? g.global_scale[0] : 1.0f;
    unsigned char* wst = smem + (size_t)xrows * XP * 2 + wave * (PPR * 32 * 16);
    float* nf4_lds = (float*)(smem + (size_t)xrows * XP * 2 + 4 * 4096);    // 16 levels behind the slabs
    if (FMT == XQ_FMT_NF4 && tid < 16) nf4_lds[tid] = kNf4Level[tid];        // ordered before its use by stage_x's barrier
    if constexpr (MR == 64) {
        constexpr int CXP = 128 + 8;                            // row pitch of an x chunk in LDS, bf16 elements
        bf16_t* xc = (bf16_t*)smem;                             // [2 buffers][64 rows][CXP]
        unsigned char* wst2 = smem + 2 * 64 * CXP * 2 + wave * (PPR * 32 * 16);
        float* nf4_2 = (float*)(smem + 2 * 64 * CXP * 2 + 4 * 4096);
        if (FMT == XQ_FMT_NF4 && tid < 16) nf4_2[tid] = kNf4Level[tid];     // ordered before its use by the first chunk's barrier
        const int xrow0 = fr < g.M ? fr : 0, xrow1 = 32 + fr < g.M ? 32 + fr : 0;
        f32x16 acc0, acc1;
#pragma unroll
        for (int q = 0; q < 16; ++q) acc0[q] = acc1[q] = 0.0f;
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            if (c < nch) {      // block-uniform
                // x chunk -> buffer c & 1.  Behind this barrier every wave is also done with chunk c - 1, whose buffer
                // the chunk after this one will overwrite.
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int row = (tid >> 4) + 16 * i;
                    if (row < g.M) *(u32x4*)(xc + ((c & 1) * 64 + row) * CXP + (tid & 15) * 8) = xcr[i];
                }
                if (c + 1 < NCH) load_xc(c + 1);
                lds_barrier();
#pragma unroll
                for (int i = 0; i < NLOAD; ++i) {
                    const int rl = RPI * i + lrow;
                    const int sw = FMT == XQ_FMT_FP8 ? (rl >> 1) & 7 : (rl >> 2) & 3;
                    *(u32x4*)(wst2 + (rl * PPR + (lpiece ^ sw)) * 16) = w[c % DC][i];
                }
                __builtin_amdgcn_wave_barrier();
                const int kc = (c_begin + c) * 128;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    uint32_t f[4];
                    if (FMT == XQ_FMT_FP8) {
                        const u32x4 t = *(const u32x4*)(wst2 + (fr * 8 + ((2 * u + fh) ^ ((fr >> 1) & 7))) * 16);
                        f[0] = t[0]; f[1] = t[1]; f[2] = t[2]; f[3] = t[3];
                    } else {
                        const u32x2 t = *(const u32x2*)(wst2 + (fr * 4 + (u ^ ((fr >> 2) & 3))) * 16 + fh * 8);
                        f[0] = t[0]; f[1] = t[1];
                    }
#pragma unroll
                    for (int v = 0; v < 2; ++v) {
                        bf16x8 wf;
                        if (FMT == XQ_FMT_FP8) {
                            wf = decode8<FMT>(f[2 * v], f[2 * v + 1], __uint_as_float(sc[c % DC][0]), 0.0f);
                        } else if (FMT == XQ_FMT_NF4) {
                            wf = decode8<FMT>(f[v], 0u, __uint_as_float(sc[c % DC][u >> 1]), 0.0f, nf4_2);
                        } else if (FMT == XQ_FMT_INT4) {
                            float sv;
                            if (int4_small_group) sv = load_scale(g.scales, ((int64_t)n * g.K + kc + 32 * u + 16 * fh + 8 * v) / g.group, g.scale_dtype);
                            else sv = g.scale_dtype == XQ_SCALE_F32 ? __uint_as_float(sc[c % DC][0]) : __uint_as_float(sc[c % DC][0] << 16);
                            wf = decode8<FMT>(f[v], 0u, sv, -8.0f * sv);
                        } else {
                            float sv;
                            if (g.scale_dtype == XQ_SCALE_E4M3) sv = e4m3_to_f32((uint8_t)(sc[c % DC][u >> 1] >> (8 * (2 * (u & 1) + fh))));
                            else sv = __uint_as_float(sc[c % DC][u]);
                            wf = decode8<FMT>(f[v], 0u, sv * gsc, 0.0f);
                        }
                        const bf16_t* xb = xc + (c & 1) * 64 * CXP + 32 * u + 16 * fh + 8 * v;
                        acc0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, *(const bf16x8*)(xb + xrow0 * CXP), acc0, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, *(const bf16x8*)(xb + xrow1 * CXP), acc1, 0, 0, 0);
                    }
                }
                __builtin_amdgcn_wave_barrier();
            }
            if (c + DC < NCH) load_chunk(c + DC);
        }
        float* out = g.partial + (int64_t)split * g.M * g.N;
#pragma unroll
        for (int hh = 0; hh < 2; ++hh) {
            const int m = hh * 32 + fr;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int nn = nbase + 8 * q4 + 4 * fh;
                if (m < g.M && nn < g.N) {
                    const f32x16& a = hh ? acc1 : acc0;
                    *(f32x4*)(out + (int64_t)m * g.N + nn) = f32x4{a[q4 * 4], a[q4 * 4 + 1], a[q4 * 4 + 2], a[q4 * 4 + 3]};
                }
            }
        }
        return;
    }
#pragma unroll
    for (int h = 0; h < NPASS; ++h) {
        if (h * 32 < g.M) {
            const int tv = h > 0 ? opaque(tid) : tid;
            if (h > 0) {
                lds_barrier();                         // every wave has read its fragments of the previous pass
                load_x(h, tv);
            }
            stage_x(h, tv);
            const int lv = tv & 63, fr = lv & 31, fh = lv >> 5, lrow = lv / PPR, lpiece = lv % PPR;
            const int xrow = h * 32 + fr < g.M ? fr : 0;
            f32x16 acc;
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[q] = 0.0f;
#pragma unroll
            for (int c = 0; c < NCH; ++c) {
                if (c < nch) {
#pragma unroll
                    for (int i = 0; i < NLOAD; ++i) {
                        const int rl = RPI * i + lrow;
                        const int sw = FMT == XQ_FMT_FP8 ? (rl >> 1) & 7 : (rl >> 2) & 3;
                        *(u32x4*)(wst + (rl * PPR + (lpiece ^ sw)) * 16) = w[c % DC][i];
                    }
                    __builtin_amdgcn_wave_barrier();
                    const int kc = (c_begin + c) * 128;
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        uint32_t f[4];
                        if (FMT == XQ_FMT_FP8) {
                            const u32x4 t = *(const u32x4*)(wst + (fr * 8 + ((2 * u + fh) ^ ((fr >> 1) & 7))) * 16);
                            f[0] = t[0]; f[1] = t[1]; f[2] = t[2]; f[3] = t[3];
                        } else {
                            const u32x2 t = *(const u32x2*)(wst + (fr * 4 + (u ^ ((fr >> 2) & 3))) * 16 + fh * 8);
                            f[0] = t[0]; f[1] = t[1];
                        }
#pragma unroll
                        for (int v = 0; v < 2; ++v) {
                            bf16x8 wf;
                            if (FMT == XQ_FMT_FP8) {
                                wf = decode8<FMT>(f[2 * v], f[2 * v + 1], __uint_as_float(sc[c % DC][0]), 0.0f);
                            } else if (FMT == XQ_FMT_NF4) {
                                wf = decode8<FMT>(f[v], 0u, __uint_as_float(sc[c % DC][u >> 1]), 0.0f, nf4_lds);   // group 64: k = 32u + ..
                            } else if (FMT == XQ_FMT_INT4) {
                                float sv;
                                if (int4_small_group) sv = load_scale(g.scales, ((int64_t)n * g.K + kc + 32 * u + 16 * fh + 8 * v) / g.group, g.scale_dtype);
                                else sv = g.scale_dtype == XQ_SCALE_F32 ? __uint_as_float(sc[c % DC][0]) : __uint_as_float(sc[c % DC][0] << 16);
                                wf = decode8<FMT>(f[v], 0u, sv, -8.0f * sv);
                            } else {
                                float sv;   // block scale 2u + fh of the chunk
                                if (g.scale_dtype == XQ_SCALE_E4M3) sv = e4m3_to_f32((uint8_t)(sc[c % DC][u >> 1] >> (8 * (2 * (u & 1) + fh))));
                                else sv = __uint_as_float(sc[c % DC][u]);
                                wf = decode8<FMT>(f[v], 0u, sv * gsc, 0.0f);
                            }
                            const bf16x8 xf = *(const bf16x8*)(xs + xrow * XP + c * 128 + 32 * u + 16 * fh + 8 * v);
                            acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf, xf, acc, 0, 0, 0);
                        }
                    }
                    __builtin_amdgcn_wave_barrier();
                }
                if (c + DC < NCH) load_chunk(c + DC);      // this chunk's registers are free (single pass only: DC == NCH otherwise)
            }
            // fp32 partial tile: lane (m = 32h + fr) holds 4 consecutive weight rows per register quad
            float* out = g.partial + (int64_t)split * g.M * g.N;
            const int m = h * 32 + fr;
#pragma unroll
            for (int q4 = 0; q4 < 4; ++q4) {
                const int nn = nbase + 8 * q4 + 4 * fh;
                if (m < g.M && nn < g.N)   // N % 16 == 0: groups of 4 columns are all in or all out
                    *(f32x4*)(out + (int64_t)m * g.N + nn) = f32x4{acc[q4 * 4], acc[q4 * 4 + 1], acc[q4 * 4 + 2], acc[q4 * 4 + 3]};
            }
        }
    }
}

// y[m][n..n+3] = sum_s part[s][m][n..] + bias + su_scale * sum_j su[m][j] * B[n][j], su = sum of the su parts.
// One wave per output row m (up to four rows per block), a lane per 4 consecutive columns.  The block's 256 B rows
// (64 B per output column and 16 ranks: twice the bytes of a row's partial tiles of eight splits) are fetched once,
// coalesced, and shared by its waves through LDS.  Loads are unconditional (indices past the end are clamped, their
// values masked to zero or never stored) and the first batch of each kind is issued before anything is waited for,
// so that the B rows, partial tiles and su parts are all in flight together.  Every sum runs in a fixed order:
// parts p = g, g+4, ... per lane group g, then the four groups; splits ascending.
// RT = 16-rank tiles of the low-rank term (0 = none); VEC = B is fp32 with r % 4 == 0 (16-byte row pieces).
// (leading scalars: see skinny_split_kernel; count_bits = splits | su_parts << 16, rank_bits = lora_f32 | r << 8 | r_pad << 16)
template <int RT, bool VEC>
__global__ void __launch_bounds__(256)
skinny_epilogue_kernel(const float* partial_, const float* su_part_, const void* lora_B_, bf16_t* y_, int32_t ldy_, int32_t M_, int32_t N_,
                       int32_t count_bits, int32_t rank_bits, SkinnyEpiArgs rest) {
    SkinnyEpiArgs g = rest;
    g.partial = partial_; g.su_part = su_part_; g.lora_B = lora_B_; g.y = y_; g.ldy = ldy_; g.M = M_; g.N = N_;
    g.splits = count_bits & 0xFFFF; g.su_parts = count_bits >> 16;
    g.lora_f32 = rank_bits & 255; g.r = (rank_bits >> 8) & 255; g.r_pad = rank_bits >> 16;
    // B tile of rank tile jt: [64 lanes][16 pieces of 4 ranks] fp32 (piece 4 e + q = ranks 4q .. 4q+3 of the lane's column
    // e), the pieces of a lane XOR-swizzled with the lane number: conflict-free 16-byte writes and reads
    __shared__ __attribute__((aligned(16))) float bt[RT > 0 ? RT : 1][64 * 64];
    const int tid = threadIdx.x, lane = tid & 63, nthreads = blockDim.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int mraw = blockIdx.y * 4 + wave;
    const int m = mraw < g.M ? mraw : g.M - 1;                   // a wave past M repeats the last row and stores nothing
    const int n0 = blockIdx.x * 256;
    int n = n0 + lane * 4;
    const bool nvalid = n < g.N;                                 // N % 4 == 0: a lane's 4 columns are all in or all out
    n = nvalid ? n : 0;
    const int j = lane & 15, pg = lane >> 4;

    // ---- issue: B pieces (piece q = 4 ranks of column n0 + q / 4), then the first 16 splits, then the first 32 su parts
    constexpr int NQ = RT > 0 ? RT * 4 : 1;                       // pieces per thread with 256 threads
    f32x4 bq[NQ];
    if (RT > 0) {
#pragma unroll
        for (int jt = 0; jt < RT; ++jt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int q = tid + i * nthreads;                 // blocks of fewer than 4 waves go round again below
                const int col = n0 + (q >> 2) < g.N ? n0 + (q >> 2) : 0, jr = jt * 16 + 4 * (q & 3);
                f32x4 t = {0.0f, 0.0f, 0.0f, 0.0f};
                if (VEC) {
                    t = *(const f32x4*)((const float*)g.lora_B + (int64_t)col * g.r + (jr < g.r ? jr : 0));
                } else {
                    // (the storage type is tested around the four loads, not around each: a branch per load would make
                    // every load wait for the one before)
                    if (g.lora_f32) {
#pragma unroll
                        for (int c = 0; c < 4; ++c) t[c] = ((const float*)g.lora_B)[(int64_t)col * g.r + (jr + c < g.r ? jr + c : 0)];
                    } else {
                        bf16_t raw[4];
#pragma unroll
                        for (int c = 0; c < 4; ++c) raw[c] = ((const bf16_t*)g.lora_B)[(int64_t)col * g.r + (jr + c < g.r ? jr + c : 0)];
#pragma unroll
                        for (int c = 0; c < 4; ++c) t[c] = bf16_to_f32(raw[c]);
                    }
                }
                bq[jt * 4 + i] = t;
            }
    }
    const float* pp = g.partial + (int64_t)m * g.N + n;
    const int64_t sstride = (int64_t)g.M * g.N;
    f32x4 pt[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) pt[u] = *(const f32x4*)(pp + (int64_t)(u < g.splits ? u : g.splits - 1) * sstride);
    const int64_t pstride = (int64_t)g.M * g.r_pad;
    float st[RT > 0 ? RT : 1][8];
#pragma unroll
    for (int jt = 0; jt < RT; ++jt)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int pi = pg + 4 * u;
            st[jt][u] = g.su_part[(int64_t)(pi < g.su_parts ? pi : g.su_parts - 1) * pstride + (int64_t)m * g.r_pad + jt * 16 + j];
        }

    asm volatile("" ::"s"(g.su_scale), "s"(g.bias));        // the arguments that did not come with the wave, in one go
    // ---- B pieces -> LDS
    if (RT > 0) {
#pragma unroll
        for (int jt = 0; jt < RT; ++jt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int q = tid + i * nthreads;
                if (q < 1024) *(f32x4*)(&bt[jt][(q >> 4) * 64 + ((q ^ (q >> 4)) & 15) * 4]) = bq[jt * 4 + i];
            }
        // blocks of one or two waves (M < 4): the pieces the first four rounds did not reach
        for (int q = tid + 4 * nthreads; q < 1024; q += nthreads) {
            const int col = n0 + (q >> 2) < g.N ? n0 + (q >> 2) : 0;
#pragma unroll
            for (int jt = 0; jt < RT; ++jt) {
                const int jr = jt * 16 + 4 * (q & 3);
                f32x4 t;
                if (g.lora_f32) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) t[c] = ((const float*)g.lora_B)[(int64_t)col * g.r + (jr + c < g.r ? jr + c : 0)];
                } else {
                    bf16_t raw[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) raw[c] = ((const bf16_t*)g.lora_B)[(int64_t)col * g.r + (jr + c < g.r ? jr + c : 0)];
#pragma unroll
                    for (int c = 0; c < 4; ++c) t[c] = bf16_to_f32(raw[c]);
                }
                *(f32x4*)(&bt[jt][(q >> 4) * 64 + ((q ^ (q >> 4)) & 15) * 4]) = t;
            }
        }
        __syncthreads();
    }

    // ---- su parts: lane (j, pg) sums parts pg, pg+4, ... of rank j of each tile
    float sv[RT > 0 ? RT : 1];
#pragma unroll
    for (int jt = 0; jt < RT; ++jt) {
        sv[jt] = 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u) sv[jt] += pg + 4 * u < g.su_parts ? st[jt][u] : 0.0f;
    }
    for (int p0 = 32; p0 < g.su_parts; p0 += 32) {
#pragma unroll
        for (int jt = 0; jt < RT; ++jt)
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int pi = p0 + pg + 4 * u;
                st[jt][u] = g.su_part[(int64_t)(pi < g.su_parts ? pi : g.su_parts - 1) * pstride + (int64_t)m * g.r_pad + jt * 16 + j];
            }
#pragma unroll
        for (int jt = 0; jt < RT; ++jt)
#pragma unroll
            for (int u = 0; u < 8; ++u) sv[jt] += p0 + pg + 4 * u < g.su_parts ? st[jt][u] : 0.0f;
    }
    // ---- partial tiles
    f32x4 o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int u = 0; u < 16; ++u) {
        if (u < g.splits) o += pt[u];                             // wave-uniform
    }
    for (int s0 = 16; s0 < g.splits; s0 += 16) {
#pragma unroll
        for (int u = 0; u < 16; ++u) pt[u] = *(const f32x4*)(pp + (int64_t)(s0 + u < g.splits ? s0 + u : g.splits - 1) * sstride);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if (s0 + u < g.splits) o += pt[u];
        }
    }
    // ---- low-rank term, 16 ranks at a time; ranks >= r hold zeros in su (and finite values in the B tile)
#pragma unroll
    for (int jt = 0; jt < RT; ++jt) {
        float tot = __shfl(sv[jt], j, 64);
        tot += __shfl(sv[jt], 16 + j, 64);
        tot += __shfl(sv[jt], 32 + j, 64);
        tot += __shfl(sv[jt], 48 + j, 64);
        tot *= g.su_scale;                                        // lane l holds su[m][jt*16 + (l & 15)], zero for ranks >= r
        if (jt * 16 + j >= g.r) tot = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            f32x4 bv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[e] = *(const f32x4*)(&bt[jt][lane * 64 + (((e * 4 + q) ^ lane) & 15) * 4]);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const float sj = __shfl(tot, 4 * q + c, 64);
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = __builtin_fmaf(sj, bv[e][c], o[e]);
            }
        }
    }
    if (!nvalid || mraw >= g.M) return;
    if (g.bias) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] += bf16_to_f32(g.bias[n + e]);
    }
    *(u32x2*)(g.y + (int64_t)m * g.ldy + n) = u32x2{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3])};
}

static inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }

// K splits for the split organisation: at most four chunks per split; more splits until the grid holds
// about two blocks per CU, never more than the 1024 blocks that are resident at once (four per CU).
struct SkinnyPlan { int splits, nch, row_blocks; };
static SkinnyPlan skinny_plan(int64_t N, int64_t K) {
    const int ct = (int)(K >> 7), rb = (int)xq_cdiv(N, 128);
    int splits = (int)xq_cdiv(ct, 4);
    while (splits < ct && (int64_t)(rb + 1) * splits < 512 && (int64_t)(rb + 1) * (splits + 1) <= 1024) ++splits;
    SkinnyPlan p;
    p.splits = splits;
    p.nch = (int)xq_cdiv(ct, splits);   // the longest split
    p.row_blocks = rb;
    return p;
}

int64_t skinny_workspace_bytes(int64_t M, int64_t N, int64_t K, int r_pad) {
    const int rp = r_pad ? r_pad : 16;
    const SkinnyPlan p = skinny_plan(N, K);
    return al256((int64_t)p.splits * M * N * 4) + al256((int64_t)p.splits * M * rp * 4) + 256;
}

bool skinny_supported(const xq_weight* w, int64_t M) {
    if (M < 1 || M > 64 || w->num_experts != 1) return false;
    if (w->format == XQ_FMT_NF4 && (w->group != 64 || w->scale_dtype != XQ_SCALE_F32)) return false;   // other nf4 storages take the tile kernels
    if (w->format != XQ_FMT_FP8 && w->layout != XQ_LAYOUT_FLAT) return false;
    if (w->cols % 128 != 0 || w->cols < 1024 || w->rows % 16 != 0) return false;
    if (w->format == XQ_FMT_INT4 && (w->group % 8 != 0)) return false;
    return true;
}

template <int FMT, int NCH>
static int launch_split_one(const SkinnyArgs& g, dim3 grid, size_t lds, hipStream_t s) {
    // at most 32 rows of 1040 B + the slabs = 49 KB: below the default dynamic LDS limit
    XQ_REQUIRE(g.ldx < (1ll << 31) && g.group < (1 << 24) && g.splits < (1 << 16) && g.chunk_q < (1 << 16),
               "xq_linear_fwd: internal error: skinny launch arguments out of range");
    const int32_t fmt_bits = g.group | g.scale_dtype << 24, split_bits = g.splits | g.su_blocks << 16, chunk_bits = g.chunk_q | g.chunk_rem << 16;
#define XQ_SPLIT_ARGS g.x, (int32_t)g.ldx, g.M, g.N, g.K, g.packed, g.scales, fmt_bits, split_bits, chunk_bits, g.xp, g
    if (g.M <= 16) skinny_split_kernel<FMT, 16, NCH><<<grid, 256, lds, s>>>(XQ_SPLIT_ARGS);
    else if (g.M <= 32) skinny_split_kernel<FMT, 32, NCH><<<grid, 256, lds, s>>>(XQ_SPLIT_ARGS);
    else skinny_split_kernel<FMT, 64, NCH><<<grid, 256, lds, s>>>(XQ_SPLIT_ARGS);
#undef XQ_SPLIT_ARGS
    return XQ_OK;
}

template <int FMT>
static int launch_split_cfg(const SkinnyArgs& g, int nch, dim3 grid, size_t lds, hipStream_t s) {
    if (nch <= 1) return launch_split_one<FMT, 1>(g, grid, lds, s);
    if (nch <= 2) return launch_split_one<FMT, 2>(g, grid, lds, s);
    return launch_split_one<FMT, 4>(g, grid, lds, s);
}

static int launch_skinny_split(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                               int lora_dtype, int r, int rp, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy,
                               void* workspace, hipStream_t stream) {
    const int64_t N = w->rows, K = w->cols;
    const SkinnyPlan p = skinny_plan(N, K);
    XQ_REQUIRE(p.nch <= 4, "xq_linear_fwd: internal error: K split too long (%d chunks)", p.nch);
    XQ_REQUIRE(rp == 0 || xq_aligned(lora_A, 16), "xq_linear_fwd: lora_A must be 16-byte aligned");
    SkinnyArgs g;
    g.x = x; g.ldx = ldx; g.M = (int)M; g.N = (int)N; g.K = (int)K;
    g.packed = (const uint8_t*)w->packed; g.scales = (const uint8_t*)w->scales; g.global_scale = w->global_scale;
    g.group = w->group; g.scale_dtype = w->scale_dtype;
    g.splits = p.splits; g.su_blocks = rp ? 1 : 0; g.xp = p.nch * 128 + 8;
    g.chunk_q = (int)(K >> 7) / p.splits; g.chunk_rem = (int)(K >> 7) % p.splits;
    g.partial = (float*)workspace;
    g.su_part = (float*)((char*)workspace + al256((int64_t)p.splits * M * N * 4));
    g.lora_A = rp ? lora_A : nullptr; g.lora_f32 = lora_dtype == XQ_DT_F32; g.r = r; g.r_pad = rp;
    const dim3 grid((unsigned)p.splits, (unsigned)(p.row_blocks + g.su_blocks));
    size_t lds = (size_t)(M < 32 ? M : 32) * g.xp * 2 + 4 * 4096 + 64;   // x slice + the four weight slabs (or the su reduction buffer) + nf4 levels
    if (M > 32 && lds < 2 * 64 * 136 * 2 + 4 * 4096 + 64) lds = 2 * 64 * 136 * 2 + 4 * 4096 + 64;   // two x chunk buffers of 64 rows

    SkinnyEpiArgs e;
    e.partial = g.partial; e.su_part = g.su_part; e.splits = p.splits; e.su_parts = rp ? p.splits : 0;
    e.M = (int)M; e.N = (int)N; e.lora_B = rp ? lora_B : nullptr; e.lora_f32 = g.lora_f32; e.r = r; e.r_pad = rp;
    e.su_scale = scaling; e.bias = bias; e.y = y; e.ldy = ldy;

    int rc;
    if (w->format == XQ_FMT_FP8) rc = launch_split_cfg<XQ_FMT_FP8>(g, p.nch, grid, lds, stream);
    else if (w->format == XQ_FMT_INT4) rc = launch_split_cfg<XQ_FMT_INT4>(g, p.nch, grid, lds, stream);
    else if (w->format == XQ_FMT_NF4) rc = launch_split_cfg<XQ_FMT_NF4>(g, p.nch, grid, lds, stream);
    else rc = launch_split_cfg<XQ_FMT_NVFP4>(g, p.nch, grid, lds, stream);
    if (rc) return rc;
    const int waves = M < 4 ? (int)M : 4;
    const dim3 egrid((unsigned)xq_cdiv(N, 256), (unsigned)xq_cdiv(M, 4));
    const bool vec = g.lora_f32 && r % 4 == 0 && xq_aligned(lora_B, 16);
    XQ_REQUIRE(ldy < (1ll << 31) && p.splits < (1 << 16), "xq_linear_fwd: internal error: skinny epilogue arguments out of range");
    const int32_t count_bits = e.splits | e.su_parts << 16, rank_bits = e.lora_f32 | e.r << 8 | e.r_pad << 16;
#define XQ_EPI_ARGS e.partial, e.su_part, e.lora_B, e.y, (int32_t)e.ldy, e.M, e.N, count_bits, rank_bits, e
#define XQ_EPI(RT)                                                                                      \
    do {                                                                                                \
        if (vec) skinny_epilogue_kernel<RT, true><<<egrid, waves * 64, 0, stream>>>(XQ_EPI_ARGS);       \
        else skinny_epilogue_kernel<RT, false><<<egrid, waves * 64, 0, stream>>>(XQ_EPI_ARGS);          \
    } while (0)
    switch (rp >> 4) {
        case 0: skinny_epilogue_kernel<0, false><<<egrid, waves * 64, 0, stream>>>(XQ_EPI_ARGS); break;
        case 1: XQ_EPI(1); break;
        case 2: XQ_EPI(2); break;
        case 3: XQ_EPI(3); break;
        default: XQ_EPI(4); break;
    }
#undef XQ_EPI
#undef XQ_EPI_ARGS
    return XQ_OK;
}

// XQ_SKINNY_ROWS=0 (or xq_set_skinny_rows(0)) keeps every skinny forward on the two-launch organisation: a process-wide
// test switch, to be set while no other thread is inside the library
static int g_skinny_rows = [] { const char* e = getenv("XQ_SKINNY_ROWS"); return e ? atoi(e) : 1; }();
void set_skinny_rows(int enabled) { g_skinny_rows = enabled; }
bool skinny_rows_enabled() { return g_skinny_rows != 0; }

int launch_skinny(const xq_weight* w, const bf16_t* x, int64_t ldx, int64_t M, const void* lora_A, const void* lora_B,
                  int lora_dtype, int r, float scaling, const bf16_t* bias, bf16_t* y, int64_t ldy, void* workspace,
                  int64_t workspace_bytes, hipStream_t stream) {
    const int64_t N = w->rows, K = w->cols;
    const int rp = r <= 0 ? 0 : ((r + 15) / 16) * 16;
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= skinny_workspace_bytes(M, N, K, rp),
               "xq_linear_fwd: workspace missing, misaligned or too small for the skinny path");
    XQ_REQUIRE(ldx % 8 == 0 && xq_aligned(x, 16) && xq_aligned(w->packed, 16), "xq_linear_fwd: operands must be 16-byte aligned");
    XQ_REQUIRE(ldy % 4 == 0 && xq_aligned(y, 8), "xq_linear_fwd: output rows must be 8-byte aligned");
    XQ_REQUIRE(rp == 0 || xq_aligned(lora_A, 4) && xq_aligned(lora_B, 4), "xq_linear_fwd: LoRA factors must be 4-byte aligned");
    // algorithmic bytes: packed weight + scales + x + y (+ LoRA factors), for the roofline figure; the timed
    // region is the whole forward (both launches)
    const double wbytes = (double)xq_packed_bytes_per_expert(w) + (double)xq_scale_bytes_per_expert(w);
    const bool timed = xq_profile_mark_begin(stream, wbytes + 2.0 * M * K + 2.0 * M * N + 4.0 * r * (K + N));
    // M <= 16: one launch, whole rows per block, where the shape and the LoRA operands fit it and a slot is free
    int rc = XQ_ERR_UNSUPPORTED;
    if (g_skinny_rows && skinny_rows_supported(w, M, lora_A, lora_B, lora_dtype, r))
        rc = launch_skinny_rows(w, x, ldx, M, lora_A, lora_B, r, scaling, bias, y, ldy, workspace, stream);
    if (rc == XQ_ERR_UNSUPPORTED)
        rc = launch_skinny_split(w, x, ldx, M, lora_A, lora_B, lora_dtype, r, rp, scaling, bias, y, ldy, workspace, stream);
    if (timed) xq_profile_mark_end(stream);
    if (rc) return rc;
    XQ_CHECK_LAUNCH("skinny forward");
    return XQ_OK;
}

}  // namespace xq
