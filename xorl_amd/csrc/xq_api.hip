// Library-level entry points: version, per-thread error text, weight validation.
#include <stdarg.h>
#include <stdio.h>

#include <algorithm>

#include "xq_common.h"

static thread_local char g_err[512] = "";

void xq_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

extern "C" const char* xq_version(void) { return "xq-hip 0.1 (gfx950)"; }
extern "C" const char* xq_last_error(void) { return g_err; }

int64_t xq_packed_bytes_per_expert(const xq_weight* w) {
    int64_t n = w->rows * w->cols;
    return w->format == XQ_FMT_FP8 ? n : n / 2;
}

static int scale_elem_bytes(int dt) { return dt == XQ_SCALE_F32 ? 4 : (dt == XQ_SCALE_BF16 ? 2 : 1); }

int64_t xq_scale_bytes_per_expert(const xq_weight* w) {
    if (w->format == XQ_FMT_FP8) return xq_cdiv(w->rows, 128) * xq_cdiv(w->cols, 128) * 4;
    return (w->rows * w->cols / w->group) * scale_elem_bytes(w->scale_dtype);
}

int xq_validate_weight(const xq_weight* w, const char* who) {
    XQ_REQUIRE(w != nullptr, "%s: weight descriptor is NULL", who);
    XQ_REQUIRE(w->format >= XQ_FMT_INT4 && w->format <= XQ_FMT_NF4, "%s: unknown format %d", who, w->format);
    XQ_REQUIRE(w->layout == XQ_LAYOUT_FLAT || w->layout == XQ_LAYOUT_GKN, "%s: unknown layout %d", who, w->layout);
    XQ_REQUIRE(w->rows >= 0 && w->cols >= 0 && w->num_experts >= 1, "%s: bad shape [%d x %lld x %lld]", who,
               w->num_experts, (long long)w->rows, (long long)w->cols);
    XQ_REQUIRE(w->rows < (1ll << 31) && w->cols < (1ll << 31), "%s: dimension exceeds 2^31", who);
    bool empty = w->rows == 0 || w->cols == 0;
    XQ_REQUIRE(empty || (w->packed && w->scales), "%s: packed/scales pointer is NULL", who);
    if (w->format == XQ_FMT_FP8) {
        XQ_REQUIRE(w->group == 128, "%s: block_fp8 block size must be 128, got %d", who, w->group);
        XQ_REQUIRE(w->scale_dtype == XQ_SCALE_F32, "%s: block_fp8 scales must be fp32", who);
        XQ_REQUIRE(empty || xq_aligned(w->scales, 4), "%s: scales not 4-byte aligned", who);
    } else {
        XQ_REQUIRE(w->group >= 2 && w->group % 2 == 0, "%s: group size must be even, got %d", who, w->group);
        int64_t gdim = w->layout == XQ_LAYOUT_FLAT ? w->cols : w->rows;
        XQ_REQUIRE(gdim % w->group == 0, "%s: grouped dimension %lld not divisible by group %d", who, (long long)gdim,
                   w->group);
        XQ_REQUIRE(w->scale_dtype >= XQ_SCALE_F32 && w->scale_dtype <= XQ_SCALE_E4M3, "%s: bad scale dtype %d", who,
                   w->scale_dtype);
        if (w->format == XQ_FMT_NVFP4) {
            XQ_REQUIRE(w->group == 16, "%s: nvfp4 block size must be 16, got %d", who, w->group);
            XQ_REQUIRE(w->global_scale != nullptr, "%s: nvfp4 needs global_scale", who);
            XQ_REQUIRE(w->scale_dtype != XQ_SCALE_BF16, "%s: nvfp4 block scales are e4m3 or fp32", who);
        } else {
            XQ_REQUIRE(w->scale_dtype != XQ_SCALE_E4M3, "%s: int4 / nf4 scales are fp32 or bf16", who);
        }
        XQ_REQUIRE(empty || xq_aligned(w->scales, scale_elem_bytes(w->scale_dtype)), "%s: scales misaligned", who);
    }
    return XQ_OK;
}

// ---------------------------------------------------------------- launch timing
// Optional per-launch timing of the fused dequant-GEMM kernel with HIP events
// recorded on the launch stream.  Off by default; the benchmark turns it on for
// its timed region.  Events are created once (no device memory is allocated).
namespace {
constexpr int kMaxProfiled = 8192;
struct ProfileState {
    bool enabled = false;
    int count = 0;
    hipEvent_t start[kMaxProfiled], stop[kMaxProfiled];
    double flops[kMaxProfiled];
    int created = 0;
} g_prof;
}  // namespace

bool xq_profile_mark_begin(hipStream_t s, double flops) {
    if (!g_prof.enabled || g_prof.count >= kMaxProfiled) return false;
    int i = g_prof.count;
    if (i >= g_prof.created) {
        if (hipEventCreate(&g_prof.start[i]) != hipSuccess || hipEventCreate(&g_prof.stop[i]) != hipSuccess) return false;
        g_prof.created = i + 1;
    }
    g_prof.flops[i] = flops;
    return hipEventRecord(g_prof.start[i], s) == hipSuccess;
}
void xq_profile_mark_end(hipStream_t s) {
    (void)hipEventRecord(g_prof.stop[g_prof.count], s);
    ++g_prof.count;
}

extern "C" int xq_profile_enable(int on) {
    g_prof.enabled = on != 0;
    g_prof.count = 0;
    return XQ_OK;
}

extern "C" int xq_profile_collect(int* n_launches, double* total_ms, double* total_flops) {
    double ms = 0.0, fl = 0.0;
    for (int i = 0; i < g_prof.count; ++i) {
        if (hipEventSynchronize(g_prof.stop[i]) != hipSuccess) {
            xq_set_error("xq_profile_collect: event synchronize failed");
            return XQ_ERR_LAUNCH;
        }
        float t = 0.0f;
        (void)hipEventElapsedTime(&t, g_prof.start[i], g_prof.stop[i]);
        ms += t;
        fl += g_prof.flops[i];
    }
    if (n_launches) *n_launches = g_prof.count;
    if (total_ms) *total_ms = ms;
    if (total_flops) *total_flops = fl;
    g_prof.count = 0;
    return XQ_OK;
}

// ---- a plain streaming read of `bytes` bytes: what the memory system gives a kernel that does nothing else.  The
// benchmark times it next to the weight-streaming forwards (same bytes, same place in a HIP graph), so that their HBM
// fraction can be read against a measured ceiling for a read of that size rather than against the data-sheet peak alone.
namespace {
__global__ void __launch_bounds__(256) read_probe_kernel(const u32x4* __restrict__ p, int64_t n16, uint32_t* __restrict__ out) {
    const int64_t stride = (int64_t)gridDim.x * 256;
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    u32x4 a = {0, 0, 0, 0};
    for (; i + 3 * stride < n16; i += 4 * stride) {            // four loads per lane in flight
        const u32x4 v0 = __builtin_nontemporal_load(p + i), v1 = __builtin_nontemporal_load(p + i + stride);
        const u32x4 v2 = __builtin_nontemporal_load(p + i + 2 * stride), v3 = __builtin_nontemporal_load(p + i + 3 * stride);
        a[0] ^= v0[0] ^ v1[0] ^ v2[0] ^ v3[0]; a[1] ^= v0[1] ^ v1[1] ^ v2[1] ^ v3[1];
        a[2] ^= v0[2] ^ v1[2] ^ v2[2] ^ v3[2]; a[3] ^= v0[3] ^ v1[3] ^ v2[3] ^ v3[3];
    }
    for (; i < n16; i += stride) {
        const u32x4 v = __builtin_nontemporal_load(p + i);
        a[0] ^= v[0]; a[1] ^= v[1]; a[2] ^= v[2]; a[3] ^= v[3];
    }
    const uint32_t x = a[0] ^ a[1] ^ a[2] ^ a[3];
    if (x == 0x9e3779b9u) out[0] = x;                          // keeps the loads; practically never taken
}
}  // namespace

extern "C" int xq_read_probe(const void* data, int64_t bytes, uint32_t* out, void* stream) {
    XQ_REQUIRE(data && out && xq_aligned(data, 16) && bytes >= 0, "xq_read_probe: NULL or misaligned buffer");
    const int64_t n16 = bytes >> 4;
    if (n16 == 0) return XQ_OK;
    const int64_t blocks = std::min<int64_t>(xq_cdiv(n16, 256 * 4), 8 * 256);
    read_probe_kernel<<<dim3((unsigned)std::max<int64_t>(blocks, 1)), 256, 0, (hipStream_t)stream>>>((const u32x4*)data, n16, out);
    XQ_CHECK_LAUNCH("xq_read_probe");
    return XQ_OK;
}
