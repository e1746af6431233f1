// Optional per-kernel-class timing with HIP events on the launch stream.  Off by default (zero cost
// beyond one branch); when on, every nc_launch_* brackets its launches with a start/stop event pair
// taken from a fixed pool.  nc_profile_read() waits for the events and sums the elapsed times.
#include "../../include/nanochat_amd.h"
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
}
