// xq_grouped_fwd_infer: the routed SwiGLU expert MLP with LoRA on block-fp8, nvfp4 or nf4 expert banks for a handful of tokens
// (decode / rollout), nothing kept for a backward.  The program is the forward of the reference's
// _MoeExpertsLoRAFunction (ops/moe/lora.py:525-713) with the rounding points of xq_grouped_fwd; what differs is the
// organisation.  With few tokens an expert sees one or two rows, so the time is the touched experts' bytes: every
// touched expert's three matrices are streamed once from HBM by blocks that each own 256 output columns and a range
// of the contraction dimension and store fp32 partial sums.  A bank matrix is [K, N] with N contiguous, so a lane keeps
// 16 output columns and walks down K -- no transposition.  One row of a unit is multiplied on the vector unit
// (v_dot2c_f32_bf16 on bf16 pairs of two weight rows: a one-row operand would leave the matrix cores idle), four rows
// by v_mfma_f32_4x4x4_16b_bf16 (four weight rows of a column against the unit's four x rows).  Two small kernels
// between and after the two streaming launches add the partial sums and the low-rank terms, apply SwiGLU and the routing
// weight and sum a token's top-k copies.  Five launches (four for up to four tokens, which need no routing launch), all
// sums in a fixed order (deterministic), nothing zeroed, no atomics on memory.
//
//   decode_route_kernel   : the touched experts' rows in units of 4 -- one block
//   decode_stream_kernel  : gate | up partial sums [bank][K slice][row][I] + x . A partial sums (blocks of their own)
//   decode_mid_kernel     : h = bf16(bf16(bf16(silu(g)) u) w), g / u = bf16(sum of slices + su . B), su = bf16(s x . A)
//   decode_stream_kernel  : down partial sums [K slice][row][H] + h . A_d partial sums
//   decode_final_kernel   : out[t] = bf16(sum over the token's copies of bf16(sum of slices + su_d . B_d))
#include "xq_lora.h"

namespace xq {
namespace {

constexpr int kDecMaxPairs = 512;       // routed copies (tokens x top-k) per call
constexpr int kDecMaxExperts = 1024;
constexpr int kDecMaxTopk = 16;
constexpr int kDecTile = 256;           // output columns of a block
constexpr int kDecChunk = 128;          // contraction rows per step of a block: one row of scale blocks
constexpr int kDecMaxChunks = 16;       // chunks per K slice at most (the slice's x rows are staged in LDS)

inline int64_t al256(int64_t b) { return (b + 255) & ~(int64_t)255; }
inline int r_pad_of(int r) { return ((r + 15) / 16) * 16; }

// routing lists in device memory: a unit is up to MR consecutive rows of one expert (units in ascending expert order):
// unit[4 u] = {expert, first row, row count, 0} (all zero past the last unit) and unit_token[4 u + m] the token of its
// row m; per row row_info[2 row] = {the routed copy it is (token * topk + slot) or -1 past the last row, its expert}; per copy
// pair_info[2 copy] = {its row or -1, its expert}.  What a block needs first sits behind one index, so that its loads
// go out together instead of one after the other's result.
// With one row per unit (direct: calls of up to four tokens) there is nothing to sort: a unit is a routed copy, its row the
// copy's number, and the kernels read the expert ids where the caller has them -- no routing launch.
struct DecLists {
    int32_t* base;
    int32_t R;
    const int32_t* selected;      // direct: [R] expert ids (NULL otherwise)
    int32_t E, topk;
    __host__ __device__ int32_t* unit() const { return base + 4; }
    __host__ __device__ int32_t* unit_token() const { return base + 4 + 4 * R; }
    __host__ __device__ int32_t* row_info() const { return base + 4 + 8 * R; }
    __host__ __device__ int32_t* pair_info() const { return base + 4 + 10 * R; }
    static int64_t bytes(int64_t R) { return (4 + 12 * R) * 4; }
};

__global__ void __launch_bounds__(512) decode_route_kernel(const int32_t* selected, int R, int E, int lg, int topk, int units_max, DecLists L) {
    const int MR = 1 << lg;                          // rows per unit
    __shared__ int32_t s_tot[2];
    __shared__ __attribute__((aligned(16))) int32_t s_cnt[kDecMaxExperts], s_begin[kDecMaxExperts], s_unit[kDecMaxExperts];
    const int t = threadIdx.x;
    for (int e = t; e < kDecMaxExperts; e += 512) s_cnt[e] = 0;
    int mine = -1;
    if (t < R) {
        const int v = selected[t];
        mine = v >= 0 && v < E ? v : -1;             // ids outside [0, E) drop their copy
    }
    __syncthreads();
    // a copy's place among its expert's rows: whichever the counter hands out.  The places differ from run to run, the
    // result does not: a row's arithmetic depends neither on its place in a unit nor on the unit's other rows, and a
    // token's copies are summed in slot order.
    int rank = 0;
    if (mine >= 0) rank = atomicAdd(&s_cnt[mine], 1);
    __syncthreads();
    for (int e = t; e < E; e += 512) {
        int b = 0, idx = 0, e2 = 0;
        for (; e2 + 4 <= e; e2 += 4) {
            const int4 c = *(const int4*)&s_cnt[e2];
            b += c.x + c.y + c.z + c.w;
            idx += ((c.x + MR - 1) >> lg) + ((c.y + MR - 1) >> lg) + ((c.z + MR - 1) >> lg) + ((c.w + MR - 1) >> lg);
        }
        for (; e2 < e; ++e2) {
            const int c = s_cnt[e2];
            b += c;
            idx += (c + MR - 1) >> lg;
        }
        s_begin[e] = b;
        s_unit[e] = idx;
        const int c = s_cnt[e];
        for (int q = 0; q * MR < c; ++q) {
            int32_t* u = L.unit() + 4 * (idx + q);
            u[0] = e;
            u[1] = b + q * MR;
            u[2] = c - q * MR < MR ? c - q * MR : MR;
            u[3] = 0;
        }
        if (e == E - 1) {
            s_tot[0] = idx + ((c + MR - 1) >> lg);   // units, rows
            s_tot[1] = b + c;
        }
    }
    __syncthreads();
    // the grid is laid out for units_max units and R rows: the others say so themselves (no rows / no copy)
    for (int u = s_tot[0] + t; u < units_max; u += 512) *(int4*)(L.unit() + 4 * u) = int4{0, 0, 0, 0};
    for (int rr = s_tot[1] + t; rr < R; rr += 512) L.row_info()[2 * rr] = -1;

    if (t < R) {
        if (mine >= 0) {
            const int rr = s_begin[mine] + rank;
            L.row_info()[2 * rr] = t;
            L.row_info()[2 * rr + 1] = mine;
            L.pair_info()[2 * t] = rr;
            L.pair_info()[2 * t + 1] = mine;
            const int u = s_unit[mine] + (rank >> lg), m = rank & (MR - 1);
            L.unit_token()[4 * u + m] = t / topk;
            // rows past a unit's own are staged as copies of its first
            if (m == 0)
                for (int q = 1; q < 4; ++q)
                    if (rank + q >= s_cnt[mine] || q >= MR) L.unit_token()[4 * u + q] = t / topk;
        } else {
            L.pair_info()[2 * t] = -1;
            L.pair_info()[2 * t + 1] = 0;
        }
    }
}

// acc += w.lo * x.lo + w.hi * x.hi on bf16 pairs (exact products, one fp32 sum); written as the instruction (the
// compiler's builtin for it has come out with wrong operand registers when fed with elements of vectors)
__device__ __forceinline__ void dec_dot2(float& acc, uint32_t w, uint32_t x) {
    asm("v_dot2c_f32_bf16 %0, %1, %2" : "+v"(acc) : "v"(w), "v"(x));
}

// sum over s < ns of p[s * stride] in ascending order, the loads sixteen at a time (slices past the end are read again
// from the last one and left out): a loop of dependent round trips would cost a memory latency per slice
__device__ __forceinline__ float sum_slices(const float* p, int64_t stride, int ns) {
    float v = 0.0f;
    for (int s0 = 0; s0 < ns; s0 += 16) {
        float t[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) t[u] = p[(int64_t)(s0 + u < ns ? s0 + u : ns - 1) * stride];
#pragma unroll
        for (int u = 0; u < 16; ++u)
            if (s0 + u < ns) v += t[u];
    }
    return v;
}
// sixteen ranks of a column of a B factor as the bf16 values the training forward multiplies with (ranks past r are
// read again from the last one; the sum leaves them out)
// (the storage type is tested once, not per element: a branch around every load would make each wait for the one before)
__device__ __forceinline__ void load_b16(float (&b)[16], const void* B, int64_t b0, int64_t ld, int j0, int r, bool f32) {
    if (f32) {
        float raw[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) raw[u] = ((const float*)B)[b0 + (int64_t)(j0 + u < r ? j0 + u : r - 1) * ld];
#pragma unroll
        for (int u = 0; u < 16; ++u) b[u] = round_bf16(raw[u]);
    } else {
        bf16_t raw[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) raw[u] = ((const bf16_t*)B)[b0 + (int64_t)(j0 + u < r ? j0 + u : r - 1) * ld];
#pragma unroll
        for (int u = 0; u < 16; ++u) b[u] = bf16_to_f32(raw[u]);
    }
}
__device__ __forceinline__ float fma_b16(float v, const float* su, const float (&b)[16], int j0, int r) {
#pragma unroll
    for (int u = 0; u < 16; ++u)
        if (j0 + u < r) v += su[j0 + u] * b[u];
    return v;
}

struct DecStream {
    const uint8_t* packed[2];       // one bank (down) or two (gate, up): block fp8 [E][K][N] e4m3 bytes; nvfp4 [E][K / 2][N]
                                    // bytes, rows 2 p (low nibble) and 2 p + 1 of a column in one byte
    const void* scales[2];          // block fp8: fp32 [E][K / 128][ceil(N / 128)]; nvfp4: e4m3 [E][K / 16][N]; nf4: fp32 [E][K / 64][N]
    const float* gs[2];             // nvfp4: the experts' global scales
    int32_t n_banks, K, N, sn;
    const bf16_t* x;                // the rows that are multiplied: token rows (by_token) or rows in expert order
    int64_t ldx;
    int32_t by_token, topk;
    int32_t cps, n_slices, n_tiles; // chunks per K slice, slices, column tiles (blockIdx.x == n_tiles: the low-rank unit)
    float* part;                    // [n_banks][n_slices][R][N]
    const void* A[2];               // LoRA A [E | 1][K][r], fp32 or bf16
    int32_t A_shared[2];
    int32_t lora_f32, r, rp;
    float* su_part;                 // [n_banks][n_slices][R][rp]
    int32_t R;
    DecLists L;
};

// One block: one unit (up to MR rows of one touched expert), one bank, one K slice, and either 256 output columns
// of the bank matrix or the x . A part of the slice.  An expert with more than MR rows is several units: their blocks
// read the same bytes at about the same time, which the caches serve.  Wave w owns rows 32 w .. +31 of every 128-row
// chunk, lane (kq = lane / 16, c = lane % 16) the row pairs 8 s + 2 kq, + 1 (s = 0..3) and columns 16 c .. + 15: a
// load instruction covers four rows' 256-byte segments, a chunk is 8 loads per lane, and the next chunk's 8 are in
// flight while one is multiplied (the first chunk's are issued before the x rows are staged).  The two rows of a pair
// are decoded to the reference's bf16 weights (e4m3 x block scale, rounded) and packed column by column, so that one
// v_dot2c per output column and x row multiplies both with the x pair of those two k, which sits in LDS as it does in
// memory.  (The register count is held down by the attribute: left alone the compiler spends every register a
// 256-thread block may have on decoding ahead.)
// nvfp4 banks (FMT = XQ_FMT_NVFP4) hold the two rows of a pair in one byte, which is the operand layout as it is: a
// lane's 16-byte load is its 16 columns of one row pair, a chunk 4 weight loads and 2 loads of e4m3 block scales (16
// columns x the wave's two 16-row groups) per lane; a byte becomes its two e2m1 values by one conversion, each times
// fl(block scale x global scale), rounded to bf16 -- the reference decoder's values.  NF4 banks (FMT = XQ_FMT_NF4,
// fp32 scales per 64 rows and column) have the same byte layout: the wave's 32 rows lie in one scale group, so a chunk
// is 4 weight loads and 4 loads of the 16 columns' scales; the 16 levels are read from a copy of the table in LDS,
// one copy per wave (16 banks: any mix of codes reads it at full rate).
template <int MR, int FMT>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(MR == 1 ? 4 : 2, 8))) decode_stream_kernel(DecStream g) {
    constexpr bool NV = FMT == XQ_FMT_NVFP4, NF = FMT == XQ_FMT_NF4, P4 = NV || NF;
    __shared__ float nf4_tab[NF ? 4 : 1][16];
    __shared__ __attribute__((aligned(16))) bf16_t xs[MR][kDecMaxChunks * kDecChunk];
    __shared__ __attribute__((aligned(16))) float red[16 * kDecTile];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = blockIdx.x, slice = blockIdx.y;
    const int li = (int)blockIdx.z / g.n_banks, bank = (int)blockIdx.z % g.n_banks;
    if (NF && tid < 64) nf4_tab[tid >> 4][tid & 15] = kNf4Level[tid & 15];    // ordered before its use by the barrier behind the x rows
    int4 unit;
    if (g.L.selected) {
        const int v = g.L.selected[li];
        unit = int4{v, li, v >= 0 && v < g.L.E ? 1 : 0, 0};
    } else {
        unit = *(const int4*)(g.L.unit() + 4 * li);
    }
    const int e = __builtin_amdgcn_readfirstlane(unit.x);
    const int row0 = __builtin_amdgcn_readfirstlane(unit.y), mc = __builtin_amdgcn_readfirstlane(unit.z);
    if (mc == 0) return;
    const int c_begin = slice * g.cps;
    const int nch = min(g.cps, g.K / kDecChunk - c_begin);           // >= 1: the launcher leaves no slice empty
    const int k0 = c_begin * kDecChunk, klen = nch * kDecChunk;
    const int64_t out_row0 = ((int64_t)bank * g.n_slices + slice) * g.R + row0;
    const bool lora_unit = tile == g.n_tiles;
    const int kq = lane >> 4, c = lane & 15;
    const int n0 = tile * kDecTile;
    const uint8_t* wbase = P4 ? g.packed[bank] + ((int64_t)e * (g.K >> 1) + ((k0 + wave * 32) >> 1)) * g.N + n0
                              : g.packed[bank] + ((int64_t)e * g.K + k0 + wave * 32) * g.N + n0;
    // MR = 1: a lane owns row pairs (dot products); MR = 4: four consecutive rows (the contraction depth of the 4x4x4 MFMA)
    constexpr bool MF = MR == 4;
    const uint32_t woff = (uint32_t)((MF ? (P4 ? 2 * kq : 4 * kq) : (P4 ? kq : 2 * kq)) * g.N + c * 16);
    // block fp8: the lane's block scale of a chunk; nvfp4: the 16 columns' e4m3 scales of the wave's two 16-row groups
    // nf4: the 16 columns' fp32 scales of the wave's 64-row group
    const uint8_t* sbase = NV ? (const uint8_t*)g.scales[bank] + ((int64_t)e * (g.K >> 4) + c_begin * 8 + wave * 2) * g.N + n0
                         : NF ? (const uint8_t*)((const float*)g.scales[bank] + ((int64_t)e * (g.K >> 6) + c_begin * 2 + (wave >> 1)) * g.N + n0)
                              : (const uint8_t*)((const float*)g.scales[bank] + ((int64_t)e * (g.K / kDecChunk) + c_begin) * g.sn + (n0 >> 7));
    const uint32_t soff = (uint32_t)(NV ? c * 16 : NF ? c * 64 : (c >> 3) * 4);
    const float gsc = NV ? g.gs[bank][e] : 1.0f;

    // a chunk's loads: block fp8 w[0..7] the eight rows and sc the block scale; nvfp4 w[0..3] the four row pairs, w[4..5]
    // the scale bytes; nf4 w[0..3] the four row pairs, w[4..7] the 16 scales
    u32x4 wa[8], wb[8];
    float sa, sb;
    auto issue = [&](u32x4(&w)[8], float& sc, int ch) {
        if (NF) {
            const uint8_t* p = wbase + (int64_t)ch * (kDecChunk / 2) * g.N;
            const uint8_t* sp = sbase + (int64_t)ch * 2 * g.N * 4 + soff;
#pragma unroll
            for (int q = 0; q < 4; ++q) w[4 + q] = *(const u32x4*)(sp + 16 * q);
#pragma unroll
            for (int st = 0; st < 4; ++st)
                w[st] = __builtin_nontemporal_load((const u32x4*)(p + (int64_t)(MF ? 8 * (st >> 1) + (st & 1) : 4 * st) * g.N + woff));
        } else if (NV) {
            const uint8_t* p = wbase + (int64_t)ch * (kDecChunk / 2) * g.N;
            const uint8_t* sp = sbase + (int64_t)ch * 8 * g.N;
            w[4] = *(const u32x4*)(sp + soff);
            w[5] = *(const u32x4*)(sp + g.N + soff);
#pragma unroll
            for (int st = 0; st < 4; ++st)
                w[st] = __builtin_nontemporal_load((const u32x4*)(p + (int64_t)(MF ? 8 * (st >> 1) + (st & 1) : 4 * st) * g.N + woff));
        } else {
            const uint8_t* p = wbase + (int64_t)ch * kDecChunk * g.N;
            sc = *(const float*)(sbase + (int64_t)ch * g.sn * 4 + soff);
            if (MF) {
#pragma unroll
                for (int i = 0; i < 8; ++i) w[i] = __builtin_nontemporal_load((const u32x4*)(p + (int64_t)(16 * (i >> 2) + (i & 3)) * g.N + woff));
            } else {
#pragma unroll
                for (int st = 0; st < 4; ++st) {
                    w[2 * st] = __builtin_nontemporal_load((const u32x4*)(p + (int64_t)(8 * st) * g.N + woff));
                    w[2 * st + 1] = __builtin_nontemporal_load((const u32x4*)(p + (int64_t)(8 * st + 1) * g.N + woff));
                }
            }
        }
    };
    if (!lora_unit) issue(wa, sa, 0);                                // block-uniform; nothing below waits for it by count

    // the unit's x rows, this slice's columns
    const int ppr = klen >> 3;                                       // 16-byte pieces per row
    for (int p = tid; p < MR * ppr; p += 256) {
        const int m = p / ppr, piece = p - m * ppr;
        const int64_t xrow = !g.by_token ? row0 + (m < mc ? m : 0) : g.L.selected ? li / g.topk : g.L.unit_token()[4 * li + m];
        *(u32x4*)(&xs[m][piece * 8]) = *(const u32x4*)(g.x + xrow * g.ldx + k0 + piece * 8);
    }
    __syncthreads();

    if (lora_unit) {
        // su part [m][j] = sum over the slice's k of x[m][k] * bf16(A[k][j]): thread (kk = tid / 16, j = tid % 16) takes
        // k = kk, kk + 16, ...; the 16 sums of a rank meet in LDS in order
        const int64_t a_base = ((int64_t)(g.A_shared[bank] ? 0 : e) * g.K + k0) * g.r;
        for (int jc = 0; jc < g.rp; jc += 16) {
            const int j = jc + (tid & 15), kk = tid >> 4;
            const int jl = j < g.r ? j : 0;
            float a_acc[MR];
#pragma unroll
            for (int m = 0; m < MR; ++m) a_acc[m] = 0.0f;
            for (int k = kk; k < klen; k += 64) {                    // klen is a multiple of 128: four loads at a time
                float a[4];
                if (g.lora_f32) {                                    // tested once per batch, not per load
                    float raw[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) raw[u] = ((const float*)g.A[bank])[a_base + (int64_t)(k + 16 * u) * g.r + jl];
#pragma unroll
                    for (int u = 0; u < 4; ++u) a[u] = round_bf16(raw[u]);
                } else {
                    bf16_t raw[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) raw[u] = ((const bf16_t*)g.A[bank])[a_base + (int64_t)(k + 16 * u) * g.r + jl];
#pragma unroll
                    for (int u = 0; u < 4; ++u) a[u] = bf16_to_f32(raw[u]);
                }
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int m = 0; m < MR; ++m) a_acc[m] += bf16_to_f32(xs[m][k + 16 * u]) * a[u];
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) red[(kk * MR + m) * 16 + (tid & 15)] = j < g.r ? a_acc[m] : 0.0f;
            __syncthreads();
            if (tid < MR * 16) {
                const int m = tid >> 4, jj = tid & 15;
                float v = 0.0f;
                for (int q = 0; q < 16; ++q) v += red[(q * MR + m) * 16 + jj];
                if (m < mc) g.su_part[(out_row0 + m) * g.rp + jc + jj] = v;
            }
            __syncthreads();
        }
        return;
    }

    float acc[MR][16];
#pragma unroll
    for (int m = 0; m < MR; ++m)
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[m][j] = 0.0f;
    // MR = 4: the unit's four x rows times four consecutive weight rows of a column are one block of v_mfma_f32_4x4x4_16b_bf16
    // (16 blocks of 4 lanes: lane j of a block gives 4 k of its column as B and 4 k of x row j as A, and receives the
    // block's four rows of its column).  A lane's 16 columns take 16 such instructions per 4 weight rows, where dot products
    // would take 128 vector instructions -- and they run beside the decode, on the matrix pipe.
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    f32x4 accq[MF ? 16 : 1];
    if (MF) {
#pragma unroll
        for (int j = 0; j < 16; ++j) accq[j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    }
    auto work4 = [&](const u32x4(&w)[8], float sc, int ch) {
        const bf16_t* xa = &xs[c & 3][ch * kDecChunk + wave * 32 + 4 * kq];
#pragma unroll
        for (int qs = 0; qs < 2; ++qs) {                             // rows 16 qs + 4 kq .. + 3 of the wave's 32
            const s16x4 av = __builtin_bit_cast(s16x4, *(const u32x2*)(xa + 16 * qs));
#pragma unroll
            for (int q = 0; q < 4; ++q) {                            // columns 4 q .. 4 q + 3 of the lane's 16
                float v[4][4];                                       // [row][column]
                if (NF) {
                    const float* tab = nf4_tab[wave];
#pragma unroll
                    for (int h = 0; h < 2; ++h)
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            const uint32_t byte = (w[2 * qs + h][q] >> (8 * b)) & 0xffu;
                            const float sv = __uint_as_float(w[4 + q][b]);
                            v[2 * h][b] = tab[byte & 15u] * sv;
                            v[2 * h + 1][b] = tab[byte >> 4] * sv;
                        }
                } else if (NV) {
                    const f32x2 s01 = e4m3x2_to_f32(w[4 + qs][q], false), s23 = e4m3x2_to_f32(w[4 + qs][q], true);
                    const float sv[4] = {s01[0] * gsc, s01[1] * gsc, s23[0] * gsc, s23[1] * gsc};
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const f32x2 v0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[2 * qs + h][q], 1.0f, 0);
                        const f32x2 v1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[2 * qs + h][q], 1.0f, 1);
                        const f32x2 v2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[2 * qs + h][q], 1.0f, 2);
                        const f32x2 v3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[2 * qs + h][q], 1.0f, 3);
                        v[2 * h][0] = v0[0] * sv[0]; v[2 * h + 1][0] = v0[1] * sv[0];
                        v[2 * h][1] = v1[0] * sv[1]; v[2 * h + 1][1] = v1[1] * sv[1];
                        v[2 * h][2] = v2[0] * sv[2]; v[2 * h + 1][2] = v2[1] * sv[2];
                        v[2 * h][3] = v3[0] * sv[3]; v[2 * h + 1][3] = v3[1] * sv[3];
                    }
                } else {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const f32x2 a01 = e4m3x2_to_f32(w[4 * qs + rr][q], false), a23 = e4m3x2_to_f32(w[4 * qs + rr][q], true);
                        v[rr][0] = a01[0] * sc; v[rr][1] = a01[1] * sc; v[rr][2] = a23[0] * sc; v[rr][3] = a23[1] * sc;
                    }
                }
#pragma unroll
                for (int b = 0; b < 4; ++b) {
                    const u32x2 bw = {pack_bf16x2(v[0][b], v[1][b]), pack_bf16x2(v[2][b], v[3][b])};
                    accq[4 * q + b] = __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(av, __builtin_bit_cast(s16x4, bw), accq[4 * q + b], 0, 0, 0);
                }
            }
        }
    };
    auto work = [&](const u32x4(&w)[8], float sc, int ch) {
        if constexpr (MF) {
            work4(w, sc, ch);
            return;
        }
        const uint32_t* xw = (const uint32_t*)&xs[0][0] + ((ch * kDecChunk + wave * 32 + 2 * kq) >> 1);
        float scl[16];                                               // nvfp4: the 16 columns' scales of the current 16-row group
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            uint32_t pk[16];
            if (NF) {
                const float* tab = nf4_tab[wave];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const uint32_t byte = (w[st][q] >> (8 * b)) & 0xffu;
                        const float sv = __uint_as_float(w[4 + q][b]);
                        pk[4 * q + b] = pack_bf16x2(tab[byte & 15u] * sv, tab[byte >> 4] * sv);
                    }
                }
            } else if (NV) {
                if ((st & 1) == 0) {
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const f32x2 s01 = e4m3x2_to_f32(w[4 + (st >> 1)][q], false), s23 = e4m3x2_to_f32(w[4 + (st >> 1)][q], true);
                        scl[4 * q + 0] = s01[0] * gsc;
                        scl[4 * q + 1] = s01[1] * gsc;
                        scl[4 * q + 2] = s23[0] * gsc;
                        scl[4 * q + 3] = s23[1] * gsc;
                    }
                }
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x2 v0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[st][q], 1.0f, 0);
                    const f32x2 v1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[st][q], 1.0f, 1);
                    const f32x2 v2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[st][q], 1.0f, 2);
                    const f32x2 v3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[st][q], 1.0f, 3);
                    pk[4 * q + 0] = pack_bf16x2(v0[0] * scl[4 * q + 0], v0[1] * scl[4 * q + 0]);
                    pk[4 * q + 1] = pack_bf16x2(v1[0] * scl[4 * q + 1], v1[1] * scl[4 * q + 1]);
                    pk[4 * q + 2] = pack_bf16x2(v2[0] * scl[4 * q + 2], v2[1] * scl[4 * q + 2]);
                    pk[4 * q + 3] = pack_bf16x2(v3[0] * scl[4 * q + 3], v3[1] * scl[4 * q + 3]);
                }
            } else {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x2 a01 = e4m3x2_to_f32(w[2 * st][q], false), a23 = e4m3x2_to_f32(w[2 * st][q], true);
                    const f32x2 b01 = e4m3x2_to_f32(w[2 * st + 1][q], false), b23 = e4m3x2_to_f32(w[2 * st + 1][q], true);
                    pk[4 * q + 0] = pack_bf16x2(a01[0] * sc, b01[0] * sc);
                    pk[4 * q + 1] = pack_bf16x2(a01[1] * sc, b01[1] * sc);
                    pk[4 * q + 2] = pack_bf16x2(a23[0] * sc, b23[0] * sc);
                    pk[4 * q + 3] = pack_bf16x2(a23[1] * sc, b23[1] * sc);
                }
            }
#pragma unroll
            for (int m = 0; m < MR; ++m) {                           // rows past the unit's own hold copies of its first: no branch here
                const uint32_t xp = xw[m * (kDecMaxChunks * kDecChunk / 2) + 4 * st];
#pragma unroll
                for (int j = 0; j < 16; ++j) dec_dot2(acc[m][j], pk[j], xp);
            }
            __builtin_amdgcn_sched_barrier(0);                       // one step's decoded pairs live at a time
        }
        // A dot result must not be read by another kind of instruction for three wait states, and the compiler does not
        // see the hazard of an instruction written in assembly: a register copy that it places at the end of a block (the
        // sums are carried through branches and loops) would read the last step's sums too early.  Nothing crosses the
        // two scheduling barriers.
        asm volatile("s_nop 3");
        __builtin_amdgcn_sched_barrier(0);
    };
    // no load sits under a condition that its wait does not share: the waits then count exactly
    int ch = 0;
    while (ch + 2 < nch) {
        issue(wb, sb, ch + 1);
        work(wa, sa, ch);
        issue(wa, sa, ch + 2);
        work(wb, sb, ch + 1);
        ch += 2;
    }
    if (nch - ch == 2) {
        issue(wb, sb, ch + 1);
        work(wa, sa, ch);
        work(wb, sb, ch + 1);
    } else {
        work(wa, sa, ch);
    }

    if (MF) {
#pragma unroll
        for (int m = 0; m < MR; ++m)
#pragma unroll
            for (int j = 0; j < 16; ++j) acc[m][j] = accq[j][m];
    }
    // the 16 partial sums of a column (4 waves x 4 row groups of a lane's 16) meet in LDS, one x row at a time
#pragma unroll
    for (int m = 0; m < MR; ++m) {
        if (m < mc) {                                                // uniform
            if (m > 0) __syncthreads();
            float* dst = red + (wave * 4 + kq) * kDecTile + c * 16;
#pragma unroll
            for (int q = 0; q < 4; ++q) *(f32x4*)(dst + 4 * q) = f32x4{acc[m][4 * q], acc[m][4 * q + 1], acc[m][4 * q + 2], acc[m][4 * q + 3]};
            __syncthreads();
            float v = 0.0f;
#pragma unroll
            for (int q = 0; q < 16; ++q) v += red[q * kDecTile + tid];
            g.part[(out_row0 + m) * g.N + n0 + tid] = v;
        }
    }
}

struct DecMid {
    const float* part;          // [2][ns][R][I]
    const float* su_part;       // [2][ns][R][rp]
    int32_t ns, R, I, r, rp;
    const void* B[2];           // LoRA B [E | 1][r][I]
    int32_t B_shared[2];
    int32_t lora_f32;
    float scaling, limit;
    const void* routing_w;      // [T * topk]
    int32_t rw_f32;
    bf16_t* h;                  // [R][I], rows in expert order
    DecLists L;
};

// one row, 256 columns: gate and up from their slices and low-rank terms, SwiGLU, the routing weight.  Everything
// that depends only on the row is requested before anything is waited for.
__global__ void __launch_bounds__(256) decode_mid_kernel(DecMid g) {
    __shared__ float su_s[2 * 64];
    const int rr = blockIdx.x, tid = threadIdx.x;
    int2 info;
    if (g.L.selected) {
        const int v = g.L.selected[rr];
        info = int2{v >= 0 && v < g.L.E ? rr : -1, v};
    } else {
        info = *(const int2*)(g.L.row_info() + 2 * rr);
    }
    const int pair = info.x, e = info.y;
    if (pair < 0) return;
    const int col = blockIdx.y * 256 + tid;
    const int64_t slice_stride = (int64_t)g.R * g.I;
    float b[2][16], gu[2];
    int64_t b0[2];
#pragma unroll
    for (int bank = 0; bank < 2; ++bank) {
        b0[bank] = (int64_t)(g.B_shared[bank] ? 0 : e) * g.r * g.I + col;
        load_b16(b[bank], g.B[bank], b0[bank], g.I, 0, g.r, g.lora_f32);
    }
    const float w = g.rw_f32 ? ((const float*)g.routing_w)[pair] : bf16_to_f32(((const bf16_t*)g.routing_w)[pair]);
#pragma unroll
    for (int bank = 0; bank < 2; ++bank) gu[bank] = sum_slices(g.part + ((int64_t)bank * g.ns * g.R + rr) * g.I + col, slice_stride, g.ns);
    if (tid < 2 * g.rp) {
        const int bank = tid / g.rp, j = tid - bank * g.rp;
        su_s[bank * 64 + j] = round_bf16(g.scaling * sum_slices(g.su_part + ((int64_t)bank * g.ns * g.R + rr) * g.rp + j, (int64_t)g.R * g.rp, g.ns));
    }
    __syncthreads();
#pragma unroll
    for (int bank = 0; bank < 2; ++bank) {
        float v = fma_b16(gu[bank], su_s + bank * 64, b[bank], 0, g.r);
        for (int j0 = 16; j0 < g.r; j0 += 16) {
            load_b16(b[bank], g.B[bank], b0[bank], g.I, j0, g.r, g.lora_f32);
            v = fma_b16(v, su_s + bank * 64, b[bank], j0, g.r);
        }
        gu[bank] = round_bf16(v);
    }
    const float gv = swiglu_clamp(gu[0], g.limit);
    const float a = round_bf16(gv * sigmoid_f32(gv));
    g.h[(int64_t)rr * g.I + col] = to_bf16(round_bf16(a * gu[1]) * w);
}

struct DecFinal {
    const float* part;          // [ns][R][H]
    const float* su_part;       // [ns][R][rp]
    int32_t ns, R, H, r, rp, topk;
    const void* B;              // LoRA B of down [E | 1][r][H]
    int32_t B_shared, lora_f32;
    float scaling;
    bf16_t* out;
    int64_t ld_out;
    DecLists L;
};

// one token, 256 columns: its copies' down projections (slices + low-rank term, rounded to bf16 each) summed in slot
// order.  Four groups of 256 threads take the slots four at a time; the rounded rows meet in LDS.
__global__ void __launch_bounds__(1024) decode_final_kernel(DecFinal g) {
    __shared__ float su_s[kDecMaxTopk * 64];
    __shared__ float d_s[kDecMaxTopk * 256];
    constexpr int NS = kDecMaxTopk / 4;                              // slots of a group at most
    const int t = blockIdx.x, tid = threadIdx.x;
    const int grp = tid >> 8, cl = tid & 255, col = blockIdx.y * 256 + cl;
    int rrs[NS], es[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int slot = grp + 4 * i;
        int2 info = int2{-1, 0};
        if (slot < g.topk) {
            const int p = t * g.topk + slot;
            if (g.L.selected) {
                const int v = g.L.selected[p];
                info = int2{v >= 0 && v < g.L.E ? p : -1, v};
            } else {
                info = *(const int2*)(g.L.pair_info() + 2 * p);
            }
        }
        rrs[i] = info.x;
        es[i] = info.y;
    }
    for (int q = tid; q < g.topk * g.rp; q += 1024) {
        const int slot = q / g.rp, j = q - slot * g.rp;
        const int p = t * g.topk + slot;
        int rr;
        if (g.L.selected) {
            const int v = g.L.selected[p];
            rr = v >= 0 && v < g.L.E ? p : -1;
        } else {
            rr = g.L.pair_info()[2 * p];
        }
        su_s[slot * 64 + j] = rr >= 0 ? round_bf16(g.scaling * sum_slices(g.su_part + (int64_t)rr * g.rp + j, (int64_t)g.R * g.rp, g.ns)) : 0.0f;
    }
    float v[NS], b[NS][16];
    int64_t b0[NS];
#pragma unroll
    for (int i = 0; i < NS; ++i) {                                   // a group's threads share rrs[i]: uniform branches
        b0[i] = (int64_t)(g.B_shared ? 0 : es[i]) * g.r * g.H + col;
        v[i] = 0.0f;
        if (rrs[i] >= 0) {
            load_b16(b[i], g.B, b0[i], g.H, 0, g.r, g.lora_f32);
            v[i] = sum_slices(g.part + (int64_t)rrs[i] * g.H + col, (int64_t)g.R * g.H, g.ns);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NS; ++i) {
        const int slot = grp + 4 * i;
        if (slot < g.topk) {
            float d = 0.0f;
            if (rrs[i] >= 0) {
                d = fma_b16(v[i], su_s + slot * 64, b[i], 0, g.r);
                for (int j0 = 16; j0 < g.r; j0 += 16) {
                    load_b16(b[i], g.B, b0[i], g.H, j0, g.r, g.lora_f32);
                    d = fma_b16(d, su_s + slot * 64, b[i], j0, g.r);
                }
                d = round_bf16(d);
            }
            d_s[slot * 256 + cl] = d;
        }
    }
    __syncthreads();
    if (grp == 0) {
        float acc = 0.0f;
        for (int slot = 0; slot < g.topk; ++slot) acc += d_s[slot * 256 + cl];     // dropped copies hold zeros
        g.out[(int64_t)t * g.ld_out + col] = to_bf16(acc);
    }
}

template <int FMT>
void launch_stream_fmt(int MR, dim3 grid, const DecStream& a, hipStream_t stream) {
    if (MR == 1) decode_stream_kernel<1, FMT><<<grid, 256, 0, stream>>>(a);
    else decode_stream_kernel<4, FMT><<<grid, 256, 0, stream>>>(a);
}
void launch_stream(int fmt, int MR, dim3 grid, const DecStream& a, hipStream_t stream) {
    if (fmt == XQ_FMT_NVFP4) launch_stream_fmt<XQ_FMT_NVFP4>(MR, grid, a, stream);
    else if (fmt == XQ_FMT_NF4) launch_stream_fmt<XQ_FMT_NF4>(MR, grid, a, stream);
    else launch_stream_fmt<XQ_FMT_FP8>(MR, grid, a, stream);
}

struct DecPlan {
    int ns_gu, cps_gu, ns_d, cps_d, units;
};

// K slices: enough blocks to fill the chip when few experts are touched (the grid is laid out for the most units that the
// call can have; blocks of units that do not exist leave at once), slices of at most kDecMaxChunks chunks
void slices_for(int chunks, int blocks_per_slice, int* ns, int* cps) {
    int want = (int)xq_cdiv(1024, blocks_per_slice);
    const int least = (int)xq_cdiv(chunks, kDecMaxChunks);
    if (want < least) want = least;
    if (want > chunks) want = chunks;
    *cps = (int)xq_cdiv(chunks, want);
    *ns = (int)xq_cdiv(chunks, *cps);
}

// units at most: every unit holds a row, and an expert's last unit alone may hold fewer than MR
DecPlan plan_for(int64_t R, int E, int64_t H, int64_t I, int MR) {
    DecPlan p;
    const int64_t most = E + R / MR;
    p.units = (int)(R < most ? R : most);
    slices_for((int)(H / kDecChunk), p.units * 2 * (int)(I / kDecTile), &p.ns_gu, &p.cps_gu);
    slices_for((int)(I / kDecChunk), p.units * (int)(H / kDecTile), &p.ns_d, &p.cps_d);
    return p;
}

// up to four tokens run one row per unit with no routing launch (measured on 128 experts, top-8, block fp8 / nvfp4: 50.6 /
// 46.1 us against 54.8 / 48.8 at four tokens; at eight 68.4 / 62.1 against 66.7 / 58.0); more tokens are grouped four
// rows to a unit
inline int rows_per_unit(int64_t n_tokens) { return n_tokens <= 4 ? 1 : 4; }

int64_t infer_workspace(int64_t R, int E, int64_t H, int64_t I, int rp, int MR) {
    const DecPlan p = plan_for(R, E, H, I, MR);
    return al256(DecLists::bytes(R)) + al256(2ll * p.ns_gu * R * I * 4) + al256(2ll * p.ns_gu * R * rp * 4) + al256(R * I * 2) +
           al256((int64_t)p.ns_d * R * H * 4) + al256((int64_t)p.ns_d * R * rp * 4) + 256;
}

bool infer_supported(const xq_weight* gate, const xq_weight* up, const xq_weight* down, int64_t n_tokens, int32_t topk, int r) {
    if (!gate || !up || !down) return false;
    const xq_weight* w[3] = {gate, up, down};
    for (int i = 0; i < 3; ++i) {
        if (w[i]->format != gate->format || !xq_aligned(w[i]->packed, 16) || !w[i]->scales) return false;
        if (w[i]->format == XQ_FMT_FP8) {
            if (w[i]->scale_dtype != XQ_SCALE_F32) return false;
        } else if (w[i]->format == XQ_FMT_NVFP4) {
            if (w[i]->layout != XQ_LAYOUT_GKN || w[i]->scale_dtype != XQ_SCALE_E4M3 || w[i]->group != 16 || !w[i]->global_scale ||
                !xq_aligned(w[i]->scales, 16))
                return false;
        } else if (w[i]->format == XQ_FMT_NF4) {
            if (w[i]->layout != XQ_LAYOUT_GKN || w[i]->scale_dtype != XQ_SCALE_F32 || w[i]->group != 64 || !xq_aligned(w[i]->scales, 16)) return false;
        } else {
            return false;
        }
    }
    const int64_t H = gate->rows, I = gate->cols;
    if (up->rows != H || up->cols != I || down->rows != I || down->cols != H) return false;
    if (H % kDecTile || I % kDecTile) return false;
    const int E = gate->num_experts;
    if (E < 1 || E > kDecMaxExperts || up->num_experts != E || down->num_experts != E) return false;
    if (topk < 1 || topk > kDecMaxTopk || n_tokens < 1 || n_tokens * topk > kDecMaxPairs) return false;
    return r >= 1 && r <= 64;
}

}  // namespace
}  // namespace xq

using namespace xq;

extern "C" int xq_grouped_infer_supported(const xq_weight* gate, const xq_weight* up, const xq_weight* down, int64_t n_tokens,
                                          int32_t topk, int r) {
    return infer_supported(gate, up, down, n_tokens, topk, r) ? 1 : 0;
}

extern "C" int64_t xq_grouped_infer_workspace_bytes(int64_t n_tokens, int32_t topk, int32_t num_experts, int64_t hidden,
                                                    int64_t intermediate, int r) {
    if (n_tokens < 1 || topk < 1 || num_experts < 1 || r < 1 || hidden < kDecChunk || intermediate < kDecChunk) return 0;
    return infer_workspace(n_tokens * topk, num_experts, hidden, intermediate, r_pad_of(r), rows_per_unit(n_tokens));
}

extern "C" int xq_grouped_fwd_infer(const xq_weight* gate, const xq_weight* up, const xq_weight* down, const xq_grouped_lora* lora,
                                    const void* hidden, int64_t ld_hidden, int64_t n_tokens, const void* routing_w, int rw_dtype,
                                    const int32_t* selected, int32_t topk, void* out, int64_t ld_out, void* workspace,
                                    int64_t workspace_bytes, void* stream_) {
    static const char* who = "xq_grouped_fwd_infer";
    XQ_REQUIRE(gate && up && down && lora, "%s: NULL descriptor", who);
    int rc;
    if ((rc = xq_validate_weight(gate, who)) || (rc = xq_validate_weight(up, who)) || (rc = xq_validate_weight(down, who))) return rc;
    XQ_REQUIRE(infer_supported(gate, up, down, n_tokens, topk, lora->r),
               "%s: takes block-fp8, nvfp4 (e4m3 block scales) or nf4 (fp32 scales, group 64) banks of one format that make an MLP (hidden and intermediate sizes multiples of %d, at most %d experts), "
               "1 to %d routed copies (tokens x top-k, top-k <= %d) and ranks 1..64; see xq_grouped_infer_supported()",
               who, kDecTile, kDecMaxExperts, kDecMaxPairs, kDecMaxTopk);
    XQ_REQUIRE(lora->dtype == XQ_DT_F32 || lora->dtype == XQ_DT_BF16, "%s: bad lora dtype", who);
    const int E = gate->num_experts;
    for (int p = 0; p < 3; ++p) {
        XQ_REQUIRE(lora->A[p] && lora->B[p], "%s: LoRA factor %d is NULL", who, p);
        XQ_REQUIRE((lora->A_experts[p] == 1 || lora->A_experts[p] == E) && (lora->B_experts[p] == 1 || lora->B_experts[p] == E),
                   "%s: a LoRA factor holds 1 (shared) or %d matrices", who, E);
    }
    XQ_REQUIRE(rw_dtype == XQ_DT_F32 || rw_dtype == XQ_DT_BF16, "%s: routing weights are fp32 or bf16", who);
    XQ_REQUIRE(hidden && routing_w && selected && out, "%s: NULL tensor", who);
    const int64_t H = gate->rows, I = gate->cols, R = n_tokens * topk;
    XQ_REQUIRE(xq_aligned(hidden, 16) && (n_tokens == 1 || ld_hidden % 8 == 0) && ld_hidden >= H && ld_out >= H,
               "%s: rows of hidden must be 16-byte aligned; row strides at least the hidden size", who);
    const int r = lora->r, rp = r_pad_of(r);
    const int MR = rows_per_unit(n_tokens);
    XQ_REQUIRE(workspace && xq_aligned(workspace, 256) && workspace_bytes >= infer_workspace(R, E, H, I, rp, MR),
               "%s: workspace missing, misaligned or smaller than xq_grouped_infer_workspace_bytes()", who);
    hipStream_t stream = (hipStream_t)stream_;
    const DecPlan pl = plan_for(R, E, H, I, MR);
    uint8_t* ws = (uint8_t*)workspace;
    int64_t used = 0;
    auto take = [&](int64_t bytes) { uint8_t* p = ws + used; used += al256(bytes); return p; };
    DecLists L{(int32_t*)take(DecLists::bytes(R)), (int32_t)R, MR == 1 ? selected : nullptr, E, topk};
    float* part_gu = (float*)take(2ll * pl.ns_gu * R * I * 4);
    float* su_gu = (float*)take(2ll * pl.ns_gu * R * rp * 4);
    bf16_t* h = (bf16_t*)take(R * I * 2);
    float* part_d = (float*)take((int64_t)pl.ns_d * R * H * 4);
    float* su_d = (float*)take((int64_t)pl.ns_d * R * rp * 4);

    if (MR > 1) {
        decode_route_kernel<<<dim3(1), 512, 0, stream>>>(selected, (int)R, E, 2, topk, pl.units, L);
        XQ_CHECK_LAUNCH(who);
    }

    const int lora_f32 = lora->dtype == XQ_DT_F32;
    DecStream s1{};
    s1.packed[0] = (const uint8_t*)gate->packed; s1.packed[1] = (const uint8_t*)up->packed;
    s1.scales[0] = gate->scales; s1.scales[1] = up->scales;
    s1.gs[0] = gate->global_scale; s1.gs[1] = up->global_scale;
    s1.n_banks = 2; s1.K = (int)H; s1.N = (int)I; s1.sn = (int)xq_cdiv(I, 128);
    s1.x = (const bf16_t*)hidden; s1.ldx = ld_hidden; s1.by_token = 1; s1.topk = topk;
    s1.cps = pl.cps_gu; s1.n_slices = pl.ns_gu; s1.n_tiles = (int)(I / kDecTile);
    s1.part = part_gu;
    s1.A[0] = lora->A[0]; s1.A[1] = lora->A[1];
    s1.A_shared[0] = lora->A_experts[0] == 1 && E > 1; s1.A_shared[1] = lora->A_experts[1] == 1 && E > 1;
    s1.lora_f32 = lora_f32; s1.r = r; s1.rp = rp; s1.su_part = su_gu; s1.R = (int)R; s1.L = L;
    const dim3 g1((unsigned)(s1.n_tiles + 1), (unsigned)pl.ns_gu, (unsigned)(pl.units * 2));
    launch_stream(gate->format, MR, g1, s1, stream);
    XQ_CHECK_LAUNCH(who);

    DecMid md{};
    md.part = part_gu; md.su_part = su_gu; md.ns = pl.ns_gu; md.R = (int)R; md.I = (int)I; md.r = r; md.rp = rp;
    md.B[0] = lora->B[0]; md.B[1] = lora->B[1];
    md.B_shared[0] = lora->B_experts[0] == 1 && E > 1; md.B_shared[1] = lora->B_experts[1] == 1 && E > 1;
    md.lora_f32 = lora_f32; md.scaling = lora->scaling; md.limit = lora->swiglu_limit > 0.0f ? lora->swiglu_limit : 0.0f;
    md.routing_w = routing_w; md.rw_f32 = rw_dtype == XQ_DT_F32; md.h = h; md.L = L;
    decode_mid_kernel<<<dim3((unsigned)R, (unsigned)(I / 256)), 256, 0, stream>>>(md);
    XQ_CHECK_LAUNCH(who);

    DecStream s2{};
    s2.packed[0] = (const uint8_t*)down->packed; s2.scales[0] = down->scales; s2.gs[0] = down->global_scale;
    s2.n_banks = 1; s2.K = (int)I; s2.N = (int)H; s2.sn = (int)xq_cdiv(H, 128);
    s2.x = h; s2.ldx = I; s2.by_token = 0; s2.topk = topk;
    s2.cps = pl.cps_d; s2.n_slices = pl.ns_d; s2.n_tiles = (int)(H / kDecTile);
    s2.part = part_d;
    s2.A[0] = lora->A[2]; s2.A_shared[0] = lora->A_experts[2] == 1 && E > 1;
    s2.lora_f32 = lora_f32; s2.r = r; s2.rp = rp; s2.su_part = su_d; s2.R = (int)R; s2.L = L;
    const dim3 g2((unsigned)(s2.n_tiles + 1), (unsigned)pl.ns_d, (unsigned)pl.units);
    launch_stream(gate->format, MR, g2, s2, stream);
    XQ_CHECK_LAUNCH(who);

    DecFinal fn{};
    fn.part = part_d; fn.su_part = su_d; fn.ns = pl.ns_d; fn.R = (int)R; fn.H = (int)H; fn.r = r; fn.rp = rp; fn.topk = topk;
    fn.B = lora->B[2]; fn.B_shared = lora->B_experts[2] == 1 && E > 1; fn.lora_f32 = lora_f32; fn.scaling = lora->scaling;
    fn.out = (bf16_t*)out; fn.ld_out = ld_out; fn.L = L;
    decode_final_kernel<<<dim3((unsigned)n_tokens, (unsigned)(H / 256)), 1024, 0, stream>>>(fn);
    XQ_CHECK_LAUNCH(who);
    return XQ_OK;
}
