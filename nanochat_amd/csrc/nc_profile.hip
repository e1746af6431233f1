// Optional per-kernel-class timing with HIP events on the launch stream.  Off by default (zero cost
// beyond one branch); when on, every nc_launch_* brackets its launches with a start/stop event pair
// taken from a fixed pool (the decode attention launch, whose duration the roofline figure is made of, gives its pair to the launch
// itself instead, see nc_prof_take).  nc_profile_read() waits for the events and sums the elapsed times.
#include "../../include/nanochat_amd.h"
#include <hip/hip_ext.h>
#include "nc_common.h"
#include "nc_kernels.h"

namespace {
constexpr int POOL = 16384;
struct Rec {
    hipEvent_t start, stop;
    int cls;
    double units;
    int64_t tag;
};
Rec g_recs[POOL];
int g_created = 0, g_used = 0;
bool g_on = false;
}  // namespace

int nc_prof_begin(int cls, double units, hipStream_t s, int64_t tag) {
    if (!g_on || cls < 0 || g_used >= POOL) return -1;
    if (g_used >= g_created) {
        if (hipEventCreate(&g_recs[g_created].start) != hipSuccess) return -1;
        if (hipEventCreate(&g_recs[g_created].stop) != hipSuccess) return -1;
        g_created++;
    }
    Rec& r = g_recs[g_used];
    r.cls = cls;
    r.units = units;
    r.tag = tag;
    (void)hipEventRecord(r.start, s);
    return g_used++;
}

// A record whose two events the caller hands to the launch itself (hipExtLaunchKernelGGL): they then hold the kernel's own begin and end
// timestamps, without the marker packets that hipEventRecord puts around a launch.  Returns false when profiling is off.
bool nc_prof_take(int cls, double units, int64_t tag, hipEvent_t* start, hipEvent_t* stop) {
    if (!g_on || cls < 0 || g_used >= POOL) return false;
    if (g_used >= g_created) {
        if (hipEventCreate(&g_recs[g_created].start) != hipSuccess) return false;
        if (hipEventCreate(&g_recs[g_created].stop) != hipSuccess) return false;
        g_created++;
    }
    Rec& r = g_recs[g_used++];
    r.cls = cls, r.units = units, r.tag = tag;
    *start = r.start, *stop = r.stop;
    return true;
}

void nc_prof_end(int slot, hipStream_t s) {
    if (slot >= 0) (void)hipEventRecord(g_recs[slot].stop, s);
}

extern "C" {

int nc_profile_enable(int on) {
    g_on = on != 0;
    g_used = 0;
    return 0;
}

static int profile_read_impl(int cls, bool by_tag, int64_t tag, double* total_ms, double* total_units, int64_t* count) {
    NC_CHECK_ARG(total_ms && total_units && count, "profile_read: null pointer");
    double ms = 0.0, units = 0.0;
    int64_t n = 0;
    for (int i = 0; i < g_used; i++) {
        if (g_recs[i].cls != cls || (by_tag && g_recs[i].tag != tag)) continue;
        if (hipEventSynchronize(g_recs[i].stop) != hipSuccess) NC_FAIL(-2, "profile_read: event wait failed");
        float t = 0.f;
        if (hipEventElapsedTime(&t, g_recs[i].start, g_recs[i].stop) != hipSuccess) NC_FAIL(-2, "profile_read: elapsed time failed");
        ms += t;
        units += g_recs[i].units;
        n++;
    }
    *total_ms = ms, *total_units = units, *count = n;
    return 0;
}

int nc_profile_read(int cls, double* total_ms, double* total_units, int64_t* count) {
    return profile_read_impl(cls, false, 0, total_ms, total_units, count);
}

int nc_profile_read_gemm(int N, int K, double* total_ms, double* total_units, int64_t* count) {
    return profile_read_impl(1, true, ((int64_t)N << 32) | (uint32_t)K, total_ms, total_units, count);
}

// ---- the matrix pipe's own ceiling on given operand bytes -------------------------------------------------
// One workgroup of 8 waves per CU; every wave issues `iters` rounds of 32 independent v_mfma_f32_16x16x128_f8f6f4 whose operands
// come from registers (loaded once from `operands`, or all zero): no memory traffic, no LDS, nothing but the matrix pipe.  The
// rate a long run of this kernel sustains is what the part's power management lets the fp8 matrix cores deliver on that data (the
// published peak is reached on all-zero operands; random e4m3 bytes settle at a lower clock), i.e. the ceiling an FP8 GEMM on such
// data is priced against.  clocks_out[2 i], [2 i + 1] (i < 4): shader-clock ticks and 100 MHz ticks that workgroup i spent in the loop.
typedef int probe_v8i __attribute__((ext_vector_type(8)));
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const probe_v8i* __restrict__ operands, int n_frags, int iters,
                                                           unsigned long long* __restrict__ clocks_out, float* __restrict__ sink) {
    probe_v8i a[4], b[2];
    const probe_v8i zero = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 4; i++) a[i] = operands ? operands[(threadIdx.x + 512u * i + 3072u * blockIdx.x) % (unsigned)n_frags] : zero;
#pragma unroll
    for (int i = 0; i < 2; i++) b[i] = operands ? operands[(threadIdx.x + 512u * (4 + i) + 3072u * blockIdx.x) % (unsigned)n_frags] : zero;
    v4f acc[32];
#pragma unroll
    for (int i = 0; i < 32; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    const unsigned long long c0 = __builtin_readcyclecounter();
    unsigned long long r0, r1;
    asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r0));
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int i = 0; i < 32; i++) asm volatile("v_mfma_f32_16x16x128_f8f6f4 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(b[i & 1]), "v"(a[i & 3]));
    }
    const unsigned long long c1 = __builtin_readcyclecounter();
    asm volatile("s_memrealtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(r1));
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < 32; i++) t += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (t == 123.456f && sink) sink[0] = t;                    // keeps the loop alive; never true for finite sums of this size
    if (threadIdx.x == 0 && blockIdx.x < 4 && clocks_out) clocks_out[2 * blockIdx.x] = c1 - c0, clocks_out[2 * blockIdx.x + 1] = r1 - r0;
}

int nc_probe_fp8_mfma_ceiling(const uint8_t* operands, int64_t operand_bytes, int iters, uint64_t* clocks_out, double* flops_out,
                              nc_stream_t stream) {
    NC_CHECK_ARG(iters > 0 && iters <= (1 << 22), "probe_fp8_mfma_ceiling: iters must be 1 .. 2^22");
    NC_CHECK_ARG(!operands || (operand_bytes >= 32 && ((uintptr_t)operands & 31) == 0), "probe_fp8_mfma_ceiling: operands need 32-byte alignment and size");
    NC_CHECK_ARG(!operands || operand_bytes / 32 < (1LL << 31), "probe_fp8_mfma_ceiling: at most 64 GiB of operand bytes");
    const int cus = nc_cu_count();
    hipLaunchKernelGGL(mfma_ceiling_kernel, dim3(cus), dim3(512), 0, (hipStream_t)stream, (const probe_v8i*)operands,
                       operands ? (int)(operand_bytes / 32) : 1, iters, (unsigned long long*)clocks_out, (float*)nullptr);
    NC_CHECK_LAUNCH("probe_fp8_mfma_ceiling");
    if (flops_out) *flops_out = (double)cus * 8.0 * 32.0 * (double)iters * 65536.0;     // 2 * 16 * 16 * 128 per instruction
    return 0;
}

// ---- what a kernel that only reads reaches on this memory ---------------------------------------------------
// Every workgroup streams a contiguous share of the buffer with 16-byte non-temporal loads, eight per thread in flight, and folds what
// it read into one word that is never stored: the duration of a launch over a buffer larger than the last-level cache is the floor of
// any kernel that has to read that many bytes once, launch and ramp included.
typedef int probe_v4i __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void stream_read_kernel(const probe_v4i* __restrict__ src, long per_wg, int* __restrict__ sink) {
    const probe_v4i* p = src + (long)blockIdx.x * per_wg;
    probe_v4i acc = {0, 0, 0, 0};
    long i = threadIdx.x;
    for (; i + 7 * 256 < per_wg; i += 8 * 256) {
        probe_v4i v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = __builtin_nontemporal_load(p + i + u * 256);
#pragma unroll
        for (int u = 0; u < 8; u++) acc ^= v[u];
    }
    for (; i < per_wg; i += 256) acc ^= __builtin_nontemporal_load(p + i);
    if (sink && (acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5eed1234 && per_wg < 0) sink[0] = 1;      // never true: keeps the loads alive
}

int nc_probe_hbm_read(const void* src, int64_t bytes, int64_t* bytes_read_out, nc_stream_t stream) {
    NC_CHECK_ARG(src && ((uintptr_t)src & 15) == 0 && bytes >= 16, "probe_hbm_read: a 16-byte aligned buffer of at least 16 bytes");
    const int grid = 8 * nc_cu_count();
    const long per_wg = (long)(bytes / 16) / grid;
    NC_CHECK_ARG(per_wg >= 1, "probe_hbm_read: at least %d bytes", 16 * grid);
    // with the profiler on, the launch carries an event pair of class 5 itself: the kernel's own begin and end, as the attention launches do
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    if (nc_prof_take(5, (double)per_wg * grid * 16, 0, &ev0, &ev1))
        hipExtLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, ev0, ev1, 0, (const probe_v4i*)src, per_wg,
                              (int*)nullptr);
    else
        hipLaunchKernelGGL(stream_read_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const probe_v4i*)src, per_wg, (int*)nullptr);
    NC_CHECK_LAUNCH("probe_hbm_read");
    if (bytes_read_out) *bytes_read_out = (int64_t)per_wg * grid * 16;
    return 0;
}
}
