// Fused dequant-GEMM tile kernel.  T = 256: 256x256x64 tiles, 8 waves (2 along M x 4
// along N, two per SIMD so one wave's LDS/VALU work hides under the other's MFMAs), each
// wave a 128x64 sub-tile of 4x2 v_mfma_f32_32x32x16_bf16 (128 fp32 accumulators) -- the
// large-M kernel.  T = 128: the same program on 128x128x64 tiles with 4 waves of 64x64
// (two blocks per CU), for problems that do not fill the chip with 256x256 tiles.
//
//   C[rows, Nout] = A[rows, Kc] . Wop (+ su[rows, r] . Lr[Nout, r]^T) (+ bias)
//
// W is a quantized [wrows, wcols] matrix: block-fp8 (e4m3 bytes, fp32 scale per
// 128x128 block), a dense 4-bit FLAT matrix (int4 / nvfp4 / nf4: two codes per byte along
// the columns, one scale per `group` consecutive columns) or, GROUPED, a 4-bit GKN matrix of an
// expert bank (two codes per byte along the rows, one scale per `group` rows of a column).
//   CONTRACT_COLS (dense forward, expert-bank dgrad):  Wop[kc][n] = W[n][kc]; the
//     decoded tile is stored in LDS as [n][kc] (kc contiguous, XOR-swizzled 16-byte
//     chunks) and read with ds_read_b128 in MFMA operand order.
//   !CONTRACT_COLS (dense dgrad, expert-bank forward): Wop[kc][n] = W[kc][n]; the
//     decoded tile is stored as it lies in memory, [kc][n], and the operand
//     fragments are read with the transposing LDS load ds_read_b64_tr_b16 -- no
//     transposed copy of the weight exists anywhere.
// Every packed code is decoded exactly once per tile, in registers, to the bf16
// value the reference decoder produces.  LDS is double buffered; the next tile's
// global loads are issued one iteration ahead, its LDS stores and decode are spread
// between the four k16 MFMA groups of the current tile, and operand fragments are
// fetched one k16 step ahead.  Operands are swapped in the MFMA (D = W_frag x
// A_frag) so that each lane ends up with 4 consecutive output columns and the
// epilogue writes 8-byte packed bf16.
//
// GROUPED: rows are in expert order; a block works on one T-row tile of one
// expert (found from the T-row tile prefix that xq_route_build emits) against
// that expert's matrix of the bank.
#pragma once

#include "xq_common.h"

namespace xq {

constexpr int F8_BK = 64;
constexpr int G256_MAX_ROUNDS = 64;   // tiles one block of the persistent program may walk (the launcher sizes the grid for it)
#ifndef XQ_SMALL_TILE_DEPTH
#define XQ_SMALL_TILE_DEPTH 2
#endif
// geometry of a T x T tile (T = 256: 8 waves, 2 x 4; T = 128: 4 waves, 2 x 2; wave tile (T/2) x 64)
template <int T>
struct Geo {
    static constexpr int BM = T, BN = T, NT = 2 * T;      // tile rows / cols, threads
    static constexpr int TM = T / 64, TN = 2;              // 32x32 MFMA tiles per wave
    static constexpr int WN = T / 64;                      // waves along N
    static constexpr int A_STAGE = BM * F8_BK;             // bf16 elements
    static constexpr int NN_PITCH = BN + 32;               // [kc][n] row pitch (T = 256: 576 B)
    static constexpr int B_STAGE_NT = BN * F8_BK;
    static constexpr int B_STAGE_NN = F8_BK * NN_PITCH;
    static constexpr int RPR = BN / 16;                    // 16-code runs per [kc] row of the tile
    static constexpr int PD = T == 256 ? 1 : XQ_SMALL_TILE_DEPTH;   // tiles in flight from global memory
    static constexpr size_t lds_bytes(bool cc) { return (size_t)(2 * A_STAGE + 2 * (cc ? B_STAGE_NT : B_STAGE_NN)) * 2; }
};

// element offset of 16-byte chunk `c` (0..7) of row `r` in a [rows][64] bf16 tile.
// gfx950 LDS has 64 banks (256 B/clk) and serves a ds_read_b128 sixteen lanes at a
// time: 16 consecutive rows (128 B each, so even/odd rows sit in different bank
// halves) must land on 8 distinct chunk slots per parity -> XOR with (r >> 1) & 7.
__device__ __forceinline__ int swz(int r, int c) { return r * 64 + ((c ^ ((r >> 1) & 7)) << 3); }

struct G256Args {
    const bf16_t* A;
    int64_t lda;
    const int32_t* a_rows;     // grouped, optional: row i of the problem is row a_rows[i] of A (the routed rows of a compact
                               // [tokens, K] matrix are read in place instead of from an expert-ordered copy)
    bf16_t* C;
    int64_t ldc;
    const uint8_t* W;          // packed codes (expert 0)
    const uint8_t* scales;     // scales (expert 0)
    const float* global_scale; // nvfp4: one per expert
    int64_t packed_stride, scale_stride;  // bytes per expert
    int32_t wrows, wcols;
    int32_t gshift;            // 4-bit: log2(group)
    int32_t scale_dtype;
    int32_t Kc, Nout;
    int64_t M;                 // total rows
    const int32_t* offsets;    // grouped: [E+1] row offsets in expert order
    const int32_t* tile_prefix;// grouped: [E+1] prefix of ceil(count / tile rows)
    int32_t num_experts;
    const bf16_t* su;          // [M, r_pad] or NULL
    const bf16_t* lora_right;  // [E][Nout, r_pad] or NULL
    int32_t r_pad;
    const bf16_t* bias;
    int32_t tiles_m, tiles_n;  // grouped: tiles_m is an upper bound
    // dense launches: ksplit > 1 divides the K-steps over gridDim.y blocks per tile; split s then writes its fp32
    // sums to partial + s * M * Nout (row pitch Nout) instead of C, and split 0 carries the low-rank term and bias
    int32_t ksplit;
    float* partial;
    // grouped block-fp8 launches over two banks of equal shape (gate and up of an expert MLP), W2 == NULL for one bank:
    //   bank forward (!CONTRACT_COLS): the output is [rows, 2 * wcols]; column tiles from ncols1 on take the second
    //     bank, its side term (su2, lora_right2) and write at their own columns -- both projections in one launch;
    //   bank dgrad (CONTRACT_COLS): the contraction runs over 2 * wcols -- the first nk1 K-steps against the first
    //     bank, the others against the second -- so dX = [dgate | dup] . [Wg ; Wu]^T leaves the kernel as one sum.
    const uint8_t* W2;
    const uint8_t* scales2;
    const bf16_t* su2;
    const bf16_t* lora_right2;
    int32_t ncols1, nk1;
    int64_t ld_su;             // row pitch of su / su2 in elements (>= r_pad)
    // gate / up / SwiGLU launch (template flag GU, dense block-fp8 forward): W is the gate weight, W2 the up weight, both
    // [Nout, Kc]; a tile holds 128 gate columns and the same 128 up columns, C is [M, 2 * Nout] (gate | up) and
    // H [M, Nout] receives bf16(silu(gate)) * up computed from the rounded outputs in the epilogue
    bf16_t* H;
    int64_t ldh;
    const bf16_t* bias2;
    // C rows start 16-byte aligned: the finished tile then leaves through LDS as whole 128-byte row pieces (the gate / up
    // launch requires it of C and H)
    int32_t wide_rows;
};

// ---------------------------------------------------------------- weight-tile loaders
// A T(n) x 64(kc) tile is split over the 2T threads as 2 runs of 16 consecutive codes
// each: run u = tid + p*2T.  CONTRACT_COLS: W row n0 + (u >> 2), columns k0 + (u&3)*16
// .. +16; otherwise W row k0 + u / (T/16), columns n0 + (u % (T/16))*16 .. +16.  load()
// fetches the packed bytes and scale(s) of K-step kt into registers; store() decodes
// one run and writes its 16 bf16 values (two 16-byte LDS stores) to the stage.

template <bool CC, int T>
__device__ __forceinline__ void store_run16(bf16_t* b, int u, const u32x4& lo, const u32x4& hi) {
    if (CC) {
        const int r = u >> 2, c = (u & 3) * 2;
        *(u32x4*)(b + swz(r, c)) = lo;
        *(u32x4*)(b + swz(r, c + 1)) = hi;
    } else {
        bf16_t* d = b + (u / Geo<T>::RPR) * Geo<T>::NN_PITCH + (u % Geo<T>::RPR) * 16;
        *(u32x4*)d = lo;
        *(u32x4*)(d + 8) = hi;
    }
}

template <bool CC, int T>
struct W256Fp8 {
    const uint8_t* src[2];
    const float* s_src[2];
    int64_t kstep;
    int scols, tid;
    u32x4 raw[2];
    float s[2];
    __device__ __forceinline__ void init(const G256Args& g, const uint8_t* pk, const uint8_t* sc, float, int n0, int tid_) {
        tid = tid_;
        scols = (g.wcols + 127) >> 7;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int u = tid + p * Geo<T>::NT;
            int wr, wc;
            if (CC) { wr = min(n0 + (u >> 2), g.wrows - 1); wc = (u & 3) * 16; }
            else { wr = u / Geo<T>::RPR; wc = min(n0 + (u % Geo<T>::RPR) * 16, g.wcols - 16); }
            src[p] = pk + (int64_t)wr * g.wcols + wc;
            s_src[p] = (const float*)sc + (CC ? (wr >> 7) * scols : (wc >> 7));
        }
        kstep = CC ? F8_BK : (int64_t)F8_BK * g.wcols;
    }
    __device__ __forceinline__ void load(int kt) {
        const int k0 = kt * F8_BK;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            raw[p] = *(const u32x4*)(src[p] + kt * kstep);
            s[p] = CC ? s_src[p][k0 >> 7] : s_src[p][(k0 >> 7) * scols];
        }
    }
    // gate / up tile: run 0 of a thread is a row of the gate weight, run 1 the same row of the up weight (LDS rows
    // tid >> 2 and 128 + (tid >> 2) of the [n][kc] tile)
    __device__ __forceinline__ void init_gu(const G256Args& g, int n0, int tid_) {
        tid = tid_;
        scols = (g.wcols + 127) >> 7;
        const int wr = min(n0 + (tid >> 2), g.wrows - 1), wc = (tid & 3) * 16;
        src[0] = g.W + (int64_t)wr * g.wcols + wc;
        src[1] = g.W2 + (int64_t)wr * g.wcols + wc;
        s_src[0] = (const float*)g.scales + (wr >> 7) * scols;
        s_src[1] = (const float*)g.scales2 + (wr >> 7) * scols;
        kstep = F8_BK;
    }
    // continue on another matrix of the same shape: byte and scale offsets between the two, both uniform
    __device__ __forceinline__ void rebase(int64_t wdelta, int64_t sdelta) {
#pragma unroll
        for (int p = 0; p < 2; ++p) { src[p] += wdelta; s_src[p] += sdelta; }
    }
    __device__ __forceinline__ void store(bf16_t* b, int p) {
        const float sc = s[p];
        u32x4 lo, hi;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x2 x0 = e4m3x2_to_f32(raw[p][i], false), x1 = e4m3x2_to_f32(raw[p][i], true);
            uint32_t v0 = pack_bf16x2(x0[0] * sc, x0[1] * sc), v1 = pack_bf16x2(x1[0] * sc, x1[1] * sc);
            if (i < 2) { lo[2 * i] = v0; lo[2 * i + 1] = v1; }
            else { hi[2 * (i - 2)] = v0; hi[2 * (i - 2) + 1] = v1; }
        }
        store_run16<CC, T>(b, tid + p * Geo<T>::NT, lo, hi);
    }
};

__device__ __forceinline__ uint32_t load_scale_raw(const uint8_t* p, int64_t idx, int dtype) {
    if (dtype == XQ_SCALE_F32) return ((const uint32_t*)p)[idx];
    if (dtype == XQ_SCALE_BF16) return ((const uint16_t*)p)[idx];
    return p[idx];
}
__device__ __forceinline__ float scale_from_raw(uint32_t raw, int dtype) {
    if (dtype == XQ_SCALE_F32) return __uint_as_float(raw);
    if (dtype == XQ_SCALE_BF16) return __uint_as_float(raw << 16);
    return e4m3_to_f32((uint8_t)raw);
}

// 8 codes of one dword -> 8 bf16 (4 packed dwords), each bf16(fl(value(code) * s)).
//   int4:  value = nib - 8.  fma(nib, s, -8s) is the same real number as (nib - 8) * s
//          (-8s is exact), so it rounds identically; only the sign of an exact zero can
//          differ from the two-step form, which no sum can see.
//   nf4:   level[nib] * s, the level read from a 64-byte copy of the table in LDS (16 banks: any mix of
//          codes in a wave is conflict free).  The copy in constant memory would be a vector memory load per
//          code, which returns in order behind the next K-step's prefetch loads and so waits for them.
//   nvfp4: v_cvt_scalef32_pk_f32_fp4 with scale 1.0 returns the exact e2m1 values of the two
//          codes of a byte (low nibble first); each is multiplied by s in fp32 and rounded
//          once, like the reference's fl(e2m1 * s).
template <int FMT>
__device__ __forceinline__ void decode8_4bit(uint32_t w, float s, uint32_t* out4, const float* nf4_lds) {
    float v[8];
    if (FMT == XQ_FMT_INT4) {
        // the nibbles become floats two at a time through the fp8 converter: a byte 0x0n read as e4m3 is n * 2^-9 for
        // every n in 0..15, and (n * 2^-9) * (512 s) is n * s exactly
        const float m8s = -8.0f * s, s512 = s * 512.0f;
        const uint32_t even = w & 0x0f0f0f0fu, odd = (w >> 4) & 0x0f0f0f0fu;
        const f32x2 e01 = e4m3x2_to_f32(even, false), e23 = e4m3x2_to_f32(even, true);
        const f32x2 o01 = e4m3x2_to_f32(odd, false), o23 = e4m3x2_to_f32(odd, true);
        v[0] = __builtin_fmaf(e01[0], s512, m8s); v[1] = __builtin_fmaf(o01[0], s512, m8s);
        v[2] = __builtin_fmaf(e01[1], s512, m8s); v[3] = __builtin_fmaf(o01[1], s512, m8s);
        v[4] = __builtin_fmaf(e23[0], s512, m8s); v[5] = __builtin_fmaf(o23[0], s512, m8s);
        v[6] = __builtin_fmaf(e23[1], s512, m8s); v[7] = __builtin_fmaf(o23[1], s512, m8s);
    } else if (FMT == XQ_FMT_NF4) {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = nf4_lds[(w >> (4 * i)) & 0xfu] * s;
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f32x2 x = i == 0 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0)
                    : i == 1 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1)
                    : i == 2 ? __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2)
                             : __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
            v[2 * i] = x[0] * s;
            v[2 * i + 1] = x[1] * s;
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) out4[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
}

template <int FMT, bool CC, int T>
struct W256Flat4 {
    const uint8_t* src[2];
    const uint8_t* sc_base;
    int64_t s_idx[2];    // scale index at K-step 0
    int64_t kstep;       // bytes per K-step
    int32_t s_kstep;     // !CC: scale entries per K-step
    int32_t col0[2];     // CC: first column of the run at K-step 0
    int gshift, sdt, tid;
    float gs;
    const float* nf4_lds;   // nf4: the 16 levels in LDS
    u32x2 raw[2];
    uint32_t sraw[2];
    __device__ __forceinline__ void init(const G256Args& g, const uint8_t* pk, const uint8_t* sc, float gscale, int n0, int tid_) {
        tid = tid_; gshift = g.gshift; sdt = g.scale_dtype; gs = gscale; sc_base = sc; nf4_lds = nullptr;
        const int spr = g.wcols >> gshift;  // scales per W row
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            const int u = tid + p * Geo<T>::NT;
            int wr, wc;
            if (CC) { wr = min(n0 + (u >> 2), g.wrows - 1); wc = (u & 3) * 16; }
            else { wr = u / Geo<T>::RPR; wc = min(n0 + (u % Geo<T>::RPR) * 16, g.wcols - 16); }
            src[p] = pk + (((int64_t)wr * g.wcols + wc) >> 1);
            s_idx[p] = (int64_t)wr * spr + (CC ? 0 : (wc >> gshift));
            col0[p] = wc;
        }
        kstep = CC ? F8_BK / 2 : (int64_t)F8_BK * g.wcols / 2;
        s_kstep = F8_BK * spr;
    }
    __device__ __forceinline__ void load(int kt) {
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            raw[p] = *(const u32x2*)(src[p] + kt * kstep);
            const int64_t si = CC ? s_idx[p] + ((col0[p] + kt * F8_BK) >> gshift) : s_idx[p] + (int64_t)kt * s_kstep;
            sraw[p] = load_scale_raw(sc_base, si, sdt);
        }
    }
    __device__ __forceinline__ void rebase(int64_t, int64_t) {}
    __device__ __forceinline__ void store(bf16_t* b, int p) {
        float s = scale_from_raw(sraw[p], sdt);
        if (FMT == XQ_FMT_NVFP4) s = s * gs;
        uint32_t lo[4], hi[4];
        decode8_4bit<FMT>(raw[p][0], s, lo, nf4_lds);
        decode8_4bit<FMT>(raw[p][1], s, hi, nf4_lds);
        store_run16<CC, T>(b, tid + p * Geo<T>::NT, u32x4{lo[0], lo[1], lo[2], lo[3]}, u32x4{hi[0], hi[1], hi[2], hi[3]});
    }
};

// 4-bit GKN matrix of an expert bank, [wrows = K, wcols = N]: byte (k / 2, n) holds rows k (low nibble) and
// k + 1 (high nibble) of column n; one scale per `group` rows per column, [K / group][N].  A thread owns one
// 16-byte piece per K-step -- 16 consecutive columns of one row pair, i.e. two 16-code runs that share their bytes
// and their 16 scales.
//   !CC (bank forward, contraction along K): pair t / RPR of the K-step's 32 row pairs, columns n0 + (t % RPR) * 16;
//   CC (bank dgrad, contraction along N): rows n0 + 2 * (t >> 2), columns k0 + (t & 3) * 16.
template <int FMT, bool CC, int T>
struct W256Gkn4 {
    const uint8_t* src;
    const uint8_t* sc_base;
    int64_t kstep;           // bytes per K-step
    int32_t wcols, row, col; // !CC: first row of the pair within the K-step; CC: global row of the pair; first column at K-step 0
    int gshift, sdt, tid;
    float gs;
    const float* nf4_lds;
    u32x4 raw;
    u32x4 s0, s1, s2, s3;    // 16 scales: 4 / 2 / 1 registers of them for fp32 / bf16 / e4m3 storage
    __device__ __forceinline__ void init(const G256Args& g, const uint8_t* pk, const uint8_t* sc, float gscale, int n0, int tid_) {
        tid = tid_; gshift = g.gshift; sdt = g.scale_dtype; gs = gscale; sc_base = sc; nf4_lds = nullptr; wcols = g.wcols;
        if (CC) {
            row = min(n0 + 2 * (tid >> 2), g.wrows - 2);
            col = (tid & 3) * 16;
            src = pk + (int64_t)(row >> 1) * g.wcols + col;
            kstep = F8_BK;
        } else {
            row = 2 * (tid / Geo<T>::RPR);
            col = min(n0 + (tid % Geo<T>::RPR) * 16, g.wcols - 16);
            src = pk + (int64_t)(row >> 1) * g.wcols + col;
            kstep = (int64_t)(F8_BK / 2) * g.wcols;
        }
    }
    __device__ __forceinline__ void load(int kt) {
        raw = *(const u32x4*)(src + kt * kstep);
        const int64_t si = CC ? (int64_t)(row >> gshift) * wcols + col + kt * F8_BK
                              : (int64_t)((kt * F8_BK + row) >> gshift) * wcols + col;
        // unconditional loads of what the widest storage needs (narrower storages read the same piece again:
        // cache hits), so that the four registers are plain values and the waits count exactly
        const int esz = sdt == XQ_SCALE_F32 ? 4 : sdt == XQ_SCALE_BF16 ? 2 : 1;
        const uint8_t* sp = sc_base + si * esz;
        const int q1 = esz >= 2 ? 16 : 0, q2 = esz == 4 ? 32 : 0, q3 = esz == 4 ? 48 : 0;
        s0 = *(const u32x4*)sp;
        s1 = *(const u32x4*)(sp + q1);
        s2 = *(const u32x4*)(sp + q2);
        s3 = *(const u32x4*)(sp + q3);
    }
    // both rows of the pair in one pass over the 16 columns, four at a time: scales and decoded values live only
    // until they are packed
    template <int SDT>
    __device__ __forceinline__ void store_both(bf16_t* b) {
        uint32_t ev[8], od[8];                       // packed bf16 pairs of the even / the odd row
#pragma unroll
        for (int q = 0; q < 4; ++q) {                // code dword q: columns 4q .. 4q + 3
            float sc[4];
            if (SDT == XQ_SCALE_F32) {
                const u32x4& f = q == 0 ? s0 : q == 1 ? s1 : q == 2 ? s2 : s3;
#pragma unroll
                for (int c = 0; c < 4; ++c) sc[c] = __uint_as_float(f[c]);
            } else if (SDT == XQ_SCALE_BF16) {
                const u32x4& h = q < 2 ? s0 : s1;
                const uint32_t d0 = h[(2 * q) & 3], d1 = h[((2 * q) & 3) + 1];
                sc[0] = __uint_as_float(d0 << 16); sc[1] = __uint_as_float(d0 & 0xffff0000u);
                sc[2] = __uint_as_float(d1 << 16); sc[3] = __uint_as_float(d1 & 0xffff0000u);
            } else {
                const f32x2 lo = e4m3x2_to_f32(s0[q], false), hi = e4m3x2_to_f32(s0[q], true);
                sc[0] = lo[0]; sc[1] = lo[1]; sc[2] = hi[0]; sc[3] = hi[1];
            }
            if (FMT == XQ_FMT_NVFP4) {
#pragma unroll
                for (int c = 0; c < 4; ++c) sc[c] = sc[c] * gs;
            }
            const uint32_t w = raw[q];
            float e[4], o[4];
            if (FMT == XQ_FMT_NVFP4) {
                const f32x2 x0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 0), x1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 1);
                const f32x2 x2 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 2), x3 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w, 1.0f, 3);
                e[0] = x0[0] * sc[0]; o[0] = x0[1] * sc[0]; e[1] = x1[0] * sc[1]; o[1] = x1[1] * sc[1];
                e[2] = x2[0] * sc[2]; o[2] = x2[1] * sc[2]; e[3] = x3[0] * sc[3]; o[3] = x3[1] * sc[3];
            } else if (FMT == XQ_FMT_INT4) {
                const uint32_t lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const float m8s = -8.0f * sc[c];
                    e[c] = __builtin_fmaf((float)((lo >> (8 * c)) & 0xffu), sc[c], m8s);
                    o[c] = __builtin_fmaf((float)((hi >> (8 * c)) & 0xffu), sc[c], m8s);
                }
            } else {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    e[c] = nf4_lds[(w >> (8 * c)) & 0xfu] * sc[c];
                    o[c] = nf4_lds[(w >> (8 * c + 4)) & 0xfu] * sc[c];
                }
            }
            ev[2 * q] = pack_bf16x2(e[0], e[1]); ev[2 * q + 1] = pack_bf16x2(e[2], e[3]);
            od[2 * q] = pack_bf16x2(o[0], o[1]); od[2 * q + 1] = pack_bf16x2(o[2], o[3]);
        }
        const u32x4 elo = {ev[0], ev[1], ev[2], ev[3]}, ehi = {ev[4], ev[5], ev[6], ev[7]};
        const u32x4 olo = {od[0], od[1], od[2], od[3]}, ohi = {od[4], od[5], od[6], od[7]};
        if (CC) {
            const int u = 2 * (tid >> 2) * 4 + (tid & 3);
            store_run16<true, T>(b, u, elo, ehi);
            store_run16<true, T>(b, u + 4, olo, ohi);
        } else {
            bf16_t* d = b + row * Geo<T>::NN_PITCH + (tid % Geo<T>::RPR) * 16;
            *(u32x4*)d = elo;
            *(u32x4*)(d + 8) = ehi;
            *(u32x4*)(d + Geo<T>::NN_PITCH) = olo;
            *(u32x4*)(d + Geo<T>::NN_PITCH + 8) = ohi;
        }
    }
    __device__ __forceinline__ void rebase(int64_t, int64_t) {}
    // the kernel stores a thread's two runs one after the other: the first call does both
    __device__ __forceinline__ void store(bf16_t* b, int p) {
        if (p != 0) return;
        if (sdt == XQ_SCALE_F32) store_both<XQ_SCALE_F32>(b);
        else if (sdt == XQ_SCALE_BF16) store_both<XQ_SCALE_BF16>(b);
        else store_both<XQ_SCALE_E4M3>(b);
    }
};

template <int FMT, bool CC, bool GROUPED, int T> struct W256Sel { using type = W256Flat4<FMT, CC, T>; };
template <int FMT, bool CC, int T> struct W256Sel<FMT, CC, true, T> { using type = W256Gkn4<FMT, CC, T>; };   // expert banks
template <bool CC, bool GROUPED, int T> struct W256Sel<XQ_FMT_FP8, CC, GROUPED, T> { using type = W256Fp8<CC, T>; };
template <bool CC, int T> struct W256Sel<XQ_FMT_FP8, CC, true, T> { using type = W256Fp8<CC, T>; };

// ---------------------------------------------------------------- the kernel
template <int FMT, bool CC, bool GROUPED, int T, bool SPLIT256 = false, bool GU = false>
__global__ void __launch_bounds__(2 * T, 2) gemm_256_kernel(G256Args g) {
    static_assert(!GU || (FMT == XQ_FMT_FP8 && CC && !GROUPED && T == 256 && !SPLIT256), "gate / up tiles: dense block-fp8 forward");
    using G = Geo<T>;
    constexpr int F8_BM = G::BM, F8_BN = G::BN, F8_A_STAGE = G::A_STAGE, F8_NN_PITCH = G::NN_PITCH;
    constexpr int TM = G::TM, TN = G::TN, NT = G::NT;
    extern __shared__ __attribute__((aligned(16))) bf16_t smem[];
    constexpr int B_STAGE = CC ? G::B_STAGE_NT : G::B_STAGE_NN;
    bf16_t* As = smem;                    // 2 stages
    bf16_t* Bs = smem + 2 * F8_A_STAGE;   // 2 stages

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / G::WN, wn = wave % G::WN;   // wave tile: rows wm*(T/2).., cols wn*64..

    // The large unsplit tile is a persistent program: block b works on the tiles b, b + gridDim.x, ... and fetches
    // the first K-step of its next tile before it multiplies the low-rank term and stores the current one, so that a
    // tile's drain and the next tile's first memory round trip overlap.  (A grid that covers every tile runs each
    // block once: the same program.)
    constexpr bool CAN_SPLIT = !GROUPED && (T == 128 || SPLIT256);
    constexpr bool PERSIST = T == 256 && !SPLIT256 && !(GROUPED && FMT != XQ_FMT_FP8);   // the GKN 4-bit loader has no registers to spare
    constexpr int MAX_ROUNDS = G256_MAX_ROUNDS;

    // ---- XCD-aware tile mapping: consecutive workgroup ids land on different XCDs, so
    // give each XCD a contiguous range of logical tiles.  Dense: walk the logical tiles
    // in groups of 4 row-tiles so concurrent tiles share operands in L2.  Grouped: walk
    // row-tile by row-tile (all column tiles of a row tile, then the next row tile of the
    // same expert) so an XCD stays on one expert's matrix.  (gridDim.x is a multiple of 8 whenever a block
    // walks more than one tile, so every tile of a block lies in the same XCD's range.)
    const int nb = g.tiles_m * g.tiles_n;
    auto tile_of = [&](int b, int& pid_m, int& pid_n) {
        const int per = nb >> 3;
        const int logical = (b < per * 8) ? (b & 7) * per + (b >> 3) : b;
        if (GROUPED) {
            pid_m = logical / g.tiles_n;
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
    };
    // Grouped: (expert, first row, end row) of every tile this block will work on, found once: thread t looks at
    // expert t (and t + NT, ...) with all loads issued together -- one memory round trip for the block instead of
    // the chain of dependent loads a binary search makes, and none per tile.  A row tile belongs to exactly one
    // expert, or to none beyond the last tile.
    __shared__ int sh_tab[GROUPED ? 3 * MAX_ROUNDS : 1];
    if constexpr (GROUPED) {
        const int first = (int)blockIdx.x, stride = (int)gridDim.x;
        const int rounds = PERSIST ? min((nb - first + stride - 1) / stride, MAX_ROUNDS) : 1;
        for (int j = tid; j < rounds; j += NT) sh_tab[3 * j] = -1;
        __syncthreads();
        for (int t = tid; t < g.num_experts; t += NT) {
            const int lo = g.tile_prefix[t], hi = g.tile_prefix[t + 1];
            const int o0 = g.offsets[t], o1 = g.offsets[t + 1];
            if (lo < hi) {
                for (int j = 0; j < rounds; ++j) {
                    int pm, pn;
                    tile_of(first + j * stride, pm, pn);
                    if (lo <= pm && pm < hi) {
                        sh_tab[3 * j] = t;
                        sh_tab[3 * j + 1] = o0 + (pm - lo) * F8_BM;
                        sh_tab[3 * j + 2] = o1;
                    }
                }
            }
        }
        __syncthreads();
    }
    // two banks (grouped block-fp8 only): a forward block past the first bank's columns works on the second bank
    constexpr bool TWO_OK = GROUPED && FMT == XQ_FMT_FP8;
    struct TileDesc {
        int e;                                          // expert (0 for a dense launch)
        int64_t row0, row_end;                          // first row of the tile, end of the rows it may read and write
        int n0, n0w, bank_width;                        // first output column; the same within its bank; columns of a bank
        const uint8_t* Wb;
        const uint8_t* Sb;
        const bf16_t* su_b;
        const bf16_t* lr_b;
    };
    auto describe = [&](int b, int round, TileDesc& t) -> bool {      // false: there is no such tile
        if (b >= nb || round >= MAX_ROUNDS) return false;
        int pid_m, pid_n;
        tile_of(b, pid_m, pid_n);
        t.e = 0;
        if constexpr (GROUPED) {
            t.e = __builtin_amdgcn_readfirstlane(sh_tab[3 * round]);
            if (t.e < 0) return false;
            t.row0 = __builtin_amdgcn_readfirstlane(sh_tab[3 * round + 1]);
            t.row_end = __builtin_amdgcn_readfirstlane(sh_tab[3 * round + 2]);
        } else {
            t.row0 = (int64_t)pid_m * F8_BM;
            t.row_end = g.M;
        }
        t.n0 = GU ? pid_n * (F8_BN / 2) : pid_n * F8_BN;      // GU: first gate (= up) column of the tile
        t.Wb = g.W; t.Sb = g.scales; t.su_b = g.su; t.lr_b = g.lora_right;
        t.n0w = t.n0;
        t.bank_width = g.Nout;
        if constexpr (TWO_OK) {
            if (g.W2 != nullptr && !CC) {
                t.bank_width = g.ncols1;
                if (t.n0 >= g.ncols1) { t.Wb = g.W2; t.Sb = g.scales2; t.su_b = g.su2; t.lr_b = g.lora_right2; t.n0w = t.n0 - g.ncols1; }
            }
        }
        return true;
    };
    // K-steps of this block: all of them, or the split's share (every split has at least one)
    // K splits: the small tile always knows them; the large tile has an instantiation of its own for them
    // (trailing rows of a launch that fill part of a round), so the unsplit one carries nothing extra
    int kt0 = 0, nk = g.Kc / F8_BK;
    const int split = CAN_SPLIT ? (int)blockIdx.y : 0;
    if (CAN_SPLIT && g.ksplit > 1) {
        const int per = (nk + g.ksplit - 1) / g.ksplit;
        kt0 = split * per;
        nk = min(per, nk - kt0);
    }

    // PD register sets hold the tiles in flight from global memory: tile j lives in set j % PD.  The large tile has
    // one (two waves per SIMD and an iteration longer than the memory latency cover it); the small tile, whose
    // iteration is a fraction of the latency, keeps PD tiles in flight.
    constexpr int PD = (GROUPED && FMT != XQ_FMT_FP8) ? 1 : Geo<T>::PD;   // the GKN 4-bit loader has no registers to spare
    static_assert(!PERSIST || PD == 1, "the persistent loop refills one register set");
    using WL = typename W256Sel<FMT, CC, GROUPED, T>::type;
    WL wls[PD];
    const float* nf4_levels = nullptr;
    if constexpr (FMT == XQ_FMT_NF4) {
        __shared__ float s_nf4[16];
        if (tid < 16) s_nf4[tid] = kNf4Level[tid];
        __syncthreads();
        nf4_levels = s_nf4;
    }
    // ---- per-thread global addresses of a tile (fixed across its K-steps except for the k offset)
    const bf16_t* a_src[4];
    int a_dst[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) a_dst[p] = swz((tid + p * NT) >> 3, (tid + p * NT) & 7);
    auto aim = [&](const TileDesc& t) {
        // the thread index as a value the optimiser cannot see through: the address arithmetic below is then done
        // per tile, where it is needed, instead of being split into tile-independent parts that would have to stay
        // in registers (or spill) across the whole main loop
        int tv = tid;
        if constexpr (PERSIST) asm volatile("" : "+v"(tv));
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int u = tv + p * NT;
            int64_t r = t.row0 + (u >> 3);
            r = r < t.row_end ? r : t.row_end - 1;
            if constexpr (GROUPED) {
                if (g.a_rows) r = g.a_rows[r];
            }
            a_src[p] = g.A + r * g.lda + (u & 7) * 8 + kt0 * F8_BK;
        }
#pragma unroll
        for (int d = 0; d < PD; ++d) {
            if constexpr (GU) wls[d].init_gu(g, t.n0, tv);
            else wls[d].init(g, t.Wb + (int64_t)t.e * g.packed_stride, t.Sb + (int64_t)t.e * g.scale_stride,
                             FMT == XQ_FMT_NVFP4 ? g.global_scale[t.e] : 1.0f, t.n0w, tv);
            wls[d].tid = tid;            // the LDS addresses of its stores do not change from tile to tile
            if constexpr (FMT == XQ_FMT_NF4) wls[d].nf4_lds = nf4_levels;
        }
    };
    // contraction over two matrices of one shape (expert-bank dgrad of gate and up; dense dgrad of gate and up): the
    // K-steps from nk1 on read the second one (same expert offset in both)
    constexpr bool TWO_K = FMT == XQ_FMT_FP8 && !GU && ((GROUPED && CC) || (!GROUPED && !CC && !SPLIT256));
    int64_t wdelta = 0, sdelta = 0;
    int nk1 = 1 << 30;
    if constexpr (TWO_K) {
        if (g.W2 != nullptr) {
            nk1 = g.nk1;
            const int64_t scols = (g.wcols + 127) >> 7;
            wdelta = (g.W2 - g.W) - (int64_t)nk1 * (CC ? F8_BK : (int64_t)F8_BK * g.wcols);
            sdelta = ((const float*)g.scales2 - (const float*)g.scales) - (int64_t)(nk1 >> 1) * (CC ? 1 : scols);
        }
    }

    u32x4 aregs[PD][4];
    auto load_a = [&](u32x4* areg, int kt) {
        const int k0 = kt * F8_BK;
#pragma unroll
        for (int p = 0; p < 4; ++p) areg[p] = *(const u32x4*)(a_src[p] + k0);
    };
    auto store_a = [&](bf16_t* a, const u32x4* areg) {
#pragma unroll
        for (int p = 0; p < 4; ++p) *(u32x4*)(a + a_dst[p]) = areg[p];
    };

    f32x16 acc[TM][TN];
    const int fr = lane & 31, fh = lane >> 5;
    auto load_frags = [&](const bf16_t* a, const bf16_t* b, int ks, bool b_is_nt, bf16x8* af, bf16x8* bfr) {
#pragma unroll
        for (int i = 0; i < TM; ++i) af[i] = *(const bf16x8*)(a + swz(wm * (T / 2) + i * 32 + fr, ks * 2 + fh));
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            if (GU) bfr[j] = *(const bf16x8*)(b + swz(j * 128 + wn * 32 + fr, ks * 2 + fh));    // j = 0 gate, 1 up: same columns
            else if (CC || b_is_nt) bfr[j] = *(const bf16x8*)(b + swz(wn * 64 + j * 32 + fr, ks * 2 + fh));
            else bfr[j] = lds_tr_frag(b, F8_NN_PITCH, ks * 16, wn * 64 + j * 32, lane);
        }
    };
    auto mma = [&](const bf16x8* af, const bf16x8* bfr) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
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
    bf16x8 af0[TM], bf0[TN], af1[TM], bf1[TN];
    auto iteration = [&](int kt, bool have_next, bool have_next2, u32x4* areg, WL& wl, int kload) {
        const bf16_t* a = As + (kt & 1) * F8_A_STAGE;
        const bf16_t* b = Bs + (kt & 1) * B_STAGE;
        bf16_t* an = As + ((kt + 1) & 1) * F8_A_STAGE;
        bf16_t* bn = Bs + ((kt + 1) & 1) * B_STAGE;
        // region 1: MFMAs of step 0 over the step-1 fragment reads, the A-tile stores and the next A loads
        mma(af0, bf0);
        load_frags(a, b, 1, false, af1, bf1);
        if (have_next) store_a(an, areg);
        if (have_next2) load_a(areg, kload);
        // interleave: one LDS read behind each of the first MFMAs, then the stores and global loads
        if (T == 256) {
            for (int q = 0; q < 6; ++q) { __builtin_amdgcn_sched_group_barrier(0x008, 1, 0); __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); }
            for (int q = 0; q < 2; ++q) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x200, 2, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        // region 2: MFMAs of step 1 over the weight decode + stores, the next weight loads, step-2 fragment reads
        mma(af1, bf1);
        if (have_next) { wl.store(bn, 0); wl.store(bn, 1); }
        if constexpr (TWO_K) {
            if (kload >= nk1 && kload - PD < nk1) wl.rebase(wdelta, sdelta);     // uniform; once per loader and tile
        }
        if (have_next2) wl.load(kt0 + kload);
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
    TileDesc cur;
    int vb = (int)blockIdx.x, round = 0;
    if (!describe(vb, 0, cur)) return;
    aim(cur);
    load_a(aregs[0], 0);
    wls[0].load(kt0);
    for (;;) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.0f;
        store_a(As, aregs[0]);
        wls[0].store(Bs, 0);
        wls[0].store(Bs, 1);
        if constexpr (PD == 1) {
            if (nk > 1) { load_a(aregs[0], 1); wls[0].load(kt0 + 1); }
            __syncthreads();
            load_frags(As, Bs, 0, false, af0, bf0);
            int kt = 0;
            for (; kt + 2 < nk; ++kt) iteration(kt, true, true, aregs[0], wls[0], kt + 2);
            if (kt + 1 < nk) { iteration(kt, true, false, aregs[0], wls[0], 0); ++kt; }
            iteration(kt, false, false, aregs[0], wls[0], 0);
        } else {
            // Tiles 1 .. PD are requested in this order, so that they also arrive in it.  Every iteration stores the
            // set of tile kt+1 and refills it with tile kt+1+PD; past the end the tile index is clamped (the last tile
            // is fetched again and stored into the stage nobody reads any more), which keeps every load unconditional.
            const int last = nk - 1;
#pragma unroll
            for (int d = 1; d <= PD; ++d) { load_a(aregs[d % PD], min(d, last)); wls[d % PD].load(kt0 + min(d, last)); }
            __syncthreads();
            load_frags(As, Bs, 0, false, af0, bf0);
            int kt = 0;
            for (; kt + PD <= nk; kt += PD) {
#pragma unroll
                for (int d = 0; d < PD; ++d)
                    iteration(kt + d, true, true, aregs[(d + 1) % PD], wls[(d + 1) % PD], min(kt + d + 1 + PD, last));
            }
#pragma unroll
            for (int d = 0; d < PD - 1; ++d)
                if (kt + d < nk) iteration(kt + d, true, true, aregs[(d + 1) % PD], wls[(d + 1) % PD], last);
        }

        // ---- the block's next tile: its first K-step is requested now and arrives while the low-rank term is
        // multiplied and the finished tile is stored (the register set and the loader are free: the pipeline is drained)
        TileDesc nx;
        bool has_next = false;
        if constexpr (PERSIST) {
            has_next = describe(vb + (int)gridDim.x, round + 1, nx);
            if (has_next) {
                aim(nx);
                load_a(aregs[0], 0);
                wls[0].load(kt0);
            }
        }

        // ---- low-rank side term: su[rows, rp] x lora_right[n, rp], both [row][k] tiles in stage 0
        if (g.r_pad > 0 && split == 0) {
            const int rp = g.r_pad, cpr = rp >> 3;  // 16-byte chunks per row
            const bf16_t* lr = cur.lr_b + (int64_t)cur.e * cur.bank_width * rp;
            for (int idx = tid; idx < F8_BM * cpr; idx += NT) {
                const int r = idx / cpr, c = idx - r * cpr;
                int64_t row = cur.row0 + r;
                row = row < cur.row_end ? row : cur.row_end - 1;
                *(u32x4*)(As + swz(r, c)) = *(const u32x4*)(cur.su_b + row * g.ld_su + c * 8);
                if constexpr (GU) {
                    // the up projection's intermediate in the second activation stage; factor rows: 128 of gate's, 128 of up's
                    *(u32x4*)(As + F8_A_STAGE + swz(r, c)) = *(const u32x4*)(g.su2 + row * g.ld_su + c * 8);
                    int n = cur.n0 + (r & 127);
                    n = n < g.Nout ? n : g.Nout - 1;
                    *(u32x4*)(Bs + swz(r, c)) = *(const u32x4*)((r < 128 ? g.lora_right : g.lora_right2) + (int64_t)n * rp + c * 8);
                } else {
                    int n = cur.n0w + r;
                    n = n < cur.bank_width ? n : cur.bank_width - 1;
                    *(u32x4*)(Bs + swz(r, c)) = *(const u32x4*)(lr + (int64_t)n * rp + c * 8);
                }
            }
            __syncthreads();
            for (int ks = 0; ks < (rp >> 4); ++ks) {
                bf16x8 af[TM], bfr[TN];
                load_frags(As, Bs, ks, true, af, bfr);
                if constexpr (GU) {
                    bf16x8 af2[TM], unused[TN];
                    load_frags(As + F8_A_STAGE, Bs, ks, true, af2, unused);
#pragma unroll
                    for (int i = 0; i < TM; ++i) {
                        acc[i][0] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[0], af[i], acc[i][0], 0, 0, 0);
                        acc[i][1] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[1], af2[i], acc[i][1], 0, 0, 0);
                    }
                } else {
                    mma(af, bfr);
                }
            }
            if (GU || g.wide_rows) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // the stages become staging areas
        }

        // ---- the finished tile.  A lane holds, per 32 x 32 MFMA tile, row fr and 4 x 4 consecutive columns; stored from
        // there, an instruction writes 16-byte pieces of 32 different rows and the memory system sees the tile as 8192
        // partial-line writes (measured: 13 % of a launch).  Instead each wave passes its (T/2) x 64 sub-tile through a
        // private LDS area ([row][64] bf16, the operand tiles' chunk swizzle; LDS operations of a wave execute in order,
        // so no barrier) and writes whole 128-byte row pieces, 8 rows per instruction.  Lanes fr and fr + 32 first swap
        // 8-byte halves (v_permlane32_swap) so that each holds 16 consecutive bytes.
        bf16_t* stg = smem + wave * (TM * 32 * 64);
        // (the lane index as a value the optimiser cannot see through: the staging addresses are then worked out here,
        // per tile, instead of being carried -- spilled -- across the main loop)
        int lv = lane;
        asm volatile("" : "+v"(lv));
        const int sfr = lv & 31, sfh = lv >> 5;
        auto stage_pair = [&](int row, int chunk, uint32_t y0, uint32_t y1, uint32_t x0, uint32_t x1) {
            // in: columns 4 fh .. + 3 of the 8-column groups 2p (y) and 2p + 1 (x); out: 8 consecutive columns of group 2p + fh
            const auto s0 = __builtin_amdgcn_permlane32_swap(y0, x0, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(y1, x1, false, false);
            *(u32x4*)(stg + swz(row, chunk)) = u32x4{s0[0], s1[0], s0[1], s1[1]};
        };

        if constexpr (GU) {
            // ---- gate / up epilogue: acc[i][0] is the gate, acc[i][1] the up projection of the same 4 x 4 columns
            // per 32-row band: the two projections as their bf16 outputs (a staged row = 32 gate columns | the same 32
            // up columns) are staged and written, then h from the rounded values goes through the same rows
            if (g.bias || g.bias2) {      // a pass of its own over the accumulators, so that the common case carries none of it
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const bf16_t* bp = j == 0 ? g.bias : g.bias2;
                    if (bp == nullptr) continue;
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        const u32x2 b = *(const u32x2*)(bp + min(cur.n0 + wn * 32 + 8 * q4 + 4 * sfh, g.Nout - 4));
#pragma unroll
                        for (int i = 0; i < TM; ++i) {
                            acc[i][j][4 * q4] += __uint_as_float(b[0] << 16); acc[i][j][4 * q4 + 1] += __uint_as_float(b[0] & 0xffff0000u);
                            acc[i][j][4 * q4 + 2] += __uint_as_float(b[1] << 16); acc[i][j][4 * q4 + 3] += __uint_as_float(b[1] & 0xffff0000u);
                        }
                    }
                }
            }
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                uint32_t gp[4][2], up[4][2], hp[4][2];
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    float gv[4], uv[4], hv[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        gv[c] = acc[i][0][4 * q4 + c];
                        uv[c] = acc[i][1][4 * q4 + c];
                        gv[c] = round_bf16(gv[c]);
                        uv[c] = round_bf16(uv[c]);
                        hv[c] = round_bf16(gv[c] * sigmoid_f32(gv[c])) * uv[c];
                    }
                    gp[q4][0] = pack_bf16x2(gv[0], gv[1]); gp[q4][1] = pack_bf16x2(gv[2], gv[3]);
                    up[q4][0] = pack_bf16x2(uv[0], uv[1]); up[q4][1] = pack_bf16x2(uv[2], uv[3]);
                    hp[q4][0] = pack_bf16x2(hv[0], hv[1]); hp[q4][1] = pack_bf16x2(hv[2], hv[3]);
                }
#pragma unroll
                for (int p = 0; p < 2; ++p) {
                    stage_pair(i * 32 + sfr, 2 * p + sfh, gp[2 * p][0], gp[2 * p][1], gp[2 * p + 1][0], gp[2 * p + 1][1]);
                    stage_pair(i * 32 + sfr, 4 + 2 * p + sfh, up[2 * p][0], up[2 * p][1], up[2 * p + 1][0], up[2 * p + 1][1]);
                }
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int rl = i * 32 + t * 8 + (lv >> 3), ch = lv & 7;
                    const u32x4 v = *(const u32x4*)(stg + swz(rl, ch));
                    const int64_t row = cur.row0 + wm * (T / 2) + rl;
                    const int n = cur.n0 + wn * 32 + (ch & 3) * 8;
                    if (row < cur.row_end && n < g.Nout) *(u32x4*)(g.C + row * g.ldc + (ch >> 2) * g.Nout + n) = v;
                }
#pragma unroll
                for (int p = 0; p < 2; ++p)
                    stage_pair(i * 32 + sfr, 2 * p + sfh, hp[2 * p][0], hp[2 * p][1], hp[2 * p + 1][0], hp[2 * p + 1][1]);
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    const int rl = i * 32 + t * 16 + (lv >> 2), ch = lv & 3;
                    const u32x4 v = *(const u32x4*)(stg + swz(rl, ch));
                    const int64_t row = cur.row0 + wm * (T / 2) + rl;
                    const int n = cur.n0 + wn * 32 + ch * 8;
                    if (row < cur.row_end && n < g.Nout) *(u32x4*)(g.H + row * g.ldh + n) = v;
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        } else {
            // ---- epilogue: lane holds, per (i, j) tile, row m = fr and 4 x 4 consecutive columns
            if (g.wide_rows && !(CAN_SPLIT && g.ksplit > 1)) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    uint32_t bw[4][2] = {};          // this lane's 16 bias values of the column tile, packed bf16
                    if (g.bias) {
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            const u32x2 b = *(const u32x2*)(g.bias + min(cur.n0 + wn * 64 + j * 32 + 8 * q4 + 4 * sfh, g.Nout - 4));
                            bw[q4][0] = b[0]; bw[q4][1] = b[1];
                        }
                    }
#pragma unroll
                    for (int i = 0; i < TM; ++i) {
                        uint32_t pk[4][2];
#pragma unroll
                        for (int q4 = 0; q4 < 4; ++q4) {
                            float v0 = acc[i][j][4 * q4], v1 = acc[i][j][4 * q4 + 1], v2 = acc[i][j][4 * q4 + 2], v3 = acc[i][j][4 * q4 + 3];
                            if (g.bias) {
                                v0 += __uint_as_float(bw[q4][0] << 16); v1 += __uint_as_float(bw[q4][0] & 0xffff0000u);
                                v2 += __uint_as_float(bw[q4][1] << 16); v3 += __uint_as_float(bw[q4][1] & 0xffff0000u);
                            }
                            pk[q4][0] = pack_bf16x2(v0, v1); pk[q4][1] = pack_bf16x2(v2, v3);
                        }
#pragma unroll
                        for (int p = 0; p < 2; ++p)
                            stage_pair(i * 32 + sfr, j * 4 + 2 * p + sfh, pk[2 * p][0], pk[2 * p][1], pk[2 * p + 1][0], pk[2 * p + 1][1]);
                    }
                }
#pragma unroll
                for (int t = 0; t < TM * 4; ++t) {
                    const int rl = t * 8 + (lv >> 3), ch = lv & 7;
                    const u32x4 v = *(const u32x4*)(stg + swz(rl, ch));
                    const int64_t row = cur.row0 + wm * (T / 2) + rl;
                    const int n = cur.n0 + wn * 64 + ch * 8;
                    if (row < cur.row_end && n < g.Nout) *(u32x4*)(g.C + row * g.ldc + n) = v;
                }
            } else
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int64_t row = cur.row0 + wm * (T / 2) + i * 32 + fr;
                if (row >= cur.row_end) continue;
                bf16_t* crow = g.C + row * g.ldc;
                float* prow = (CAN_SPLIT && g.ksplit > 1) ? g.partial + ((int64_t)split * g.M + row) * g.Nout : nullptr;
#pragma unroll
                for (int j = 0; j < TN; ++j) {
#pragma unroll
                    for (int q4 = 0; q4 < 4; ++q4) {
                        const int n = cur.n0 + wn * 64 + j * 32 + 8 * q4 + 4 * fh;
                        if (n >= g.Nout) continue;  // Nout % 16 == 0: groups of 4 are all in or all out
                        float v0 = acc[i][j][4 * q4], v1 = acc[i][j][4 * q4 + 1], v2 = acc[i][j][4 * q4 + 2], v3 = acc[i][j][4 * q4 + 3];
                        if (g.bias && split == 0) {
                            v0 += bf16_to_f32(g.bias[n]); v1 += bf16_to_f32(g.bias[n + 1]);
                            v2 += bf16_to_f32(g.bias[n + 2]); v3 += bf16_to_f32(g.bias[n + 3]);
                        }
                        if (prow) *(f32x4*)(prow + n) = f32x4{v0, v1, v2, v3};
                        else *(u32x2*)(crow + n) = u32x2{pack_bf16x2(v0, v1), pack_bf16x2(v2, v3)};
                    }
                }
            }
        }
        if (!has_next) break;
        cur = nx;
        vb += (int)gridDim.x;
        ++round;
        __syncthreads();      // the low-rank fragments of stage 0 have been read before the next tile is stored there
    }
}

// C[row][n] = bf16(partial[0][row][n] + partial[1][row][n] + ...), splits added in index order; a thread per 4 columns
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float* __restrict__ partial, int ksplit, int64_t M, int Nout,
                                                            bf16_t* __restrict__ C, int64_t ldc) {
    const int64_t quads = (int64_t)(Nout >> 2), idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * quads) return;
    const int64_t row = idx / quads, n = (idx - row * quads) << 2;
    const float* p = partial + row * Nout + n;
    f32x4 acc = *(const f32x4*)p;
    for (int s = 1; s < ksplit; ++s) {
        const f32x4 v = *(const f32x4*)(p + (int64_t)s * M * Nout);
        acc[0] += v[0]; acc[1] += v[1]; acc[2] += v[2]; acc[3] += v[3];
    }
    *(u32x2*)(C + row * ldc + n) = u32x2{pack_bf16x2(acc[0], acc[1]), pack_bf16x2(acc[2], acc[3])};
}

}  // namespace xq
