// Tensorwise dynamic e4m3 quantization: amax reduce, then scale + saturate + convert.
// Replaces the eight eager ops of nanochat/fp8.py:91-106 (_to_fp8).
//
// Bit contract: amax in fp32; scale = fp32(448 / max(fp64(amax), 1e-12)); y = fp32(x) * scale
// (one fp32 rounding); clamp to +-448; round to nearest even into OCP e4m3fn; inv = 1.0f / scale
// with an IEEE divide.  HBM traffic: the amax pass reads the tensor once, the convert pass reads
// it again (normally from L2 / infinity cache) and writes one byte per element.
#include <atomic>
#include "nc_common.h"
#include "nc_kernels.h"

// ---------------------------------------------------------------- pass 1: amax
// bf16: |x| ordering equals integer ordering of the low 15 bits; fp32 likewise on 31 bits.
// Each thread takes 16-byte vectors grid-stride; one atomicMax per block on the fp32 bit pattern.
template <bool IS_BF16>
__global__ __launch_bounds__(256) void amax_kernel(const void* __restrict__ x, int64_t n, uint32_t* __restrict__ amax_bits) {
    constexpr int PER_VEC = IS_BF16 ? 8 : 4;
    const int64_t nvec = n / PER_VEC;
    const uint4* xv = (const uint4*)x;
    uint32_t m = 0;
    auto take = [&](const uint4& v) {
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (IS_BF16) {
                uint32_t lo = (w[j] & 0x7fffu) << 16, hi = w[j] & 0x7fff0000u;
                m = m > lo ? m : lo;
                m = m > hi ? m : hi;
            } else {
                uint32_t a = w[j] & 0x7fffffffu;
                m = m > a ? m : a;
            }
        }
    };
    // four 16-byte loads in flight per thread
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i + 3 * stride < nvec; i += 4 * stride) {
        const uint4 v0 = xv[i], v1 = xv[i + stride], v2 = xv[i + 2 * stride], v3 = xv[i + 3 * stride];
        take(v0), take(v1), take(v2), take(v3);
    }
    for (; i < nvec; i += stride) take(xv[i]);
    // tail elements (n not a multiple of the vector width)
    if (blockIdx.x == 0) {
        for (int64_t i = nvec * PER_VEC + threadIdx.x; i < n; i += blockDim.x) {
            uint32_t a = IS_BF16 ? (((uint32_t)((const bf16_t*)x)[i] & 0x7fffu) << 16)
                                 : (((const uint32_t*)x)[i] & 0x7fffffffu);
            m = m > a ? m : a;
        }
    }
    m = wave_max_u32(m);
    __shared__ uint32_t red[4];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    if (lane == 0) red[w] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = red[0];
        for (int i = 1; i < 4; i++) t = t > red[i] ? t : red[i];
        // atomics on one word serialize: skip the ones that cannot change it
        if (t > __hip_atomic_load(amax_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) atomicMax(amax_bits, t);
    }
}

// ---------------------------------------------------------------- pass 2: convert
template <bool IS_BF16, bool HW_CVT, int FMT = 0>
__global__ __launch_bounds__(256) void convert_kernel(const void* __restrict__ x, int64_t n, const uint32_t* __restrict__ amax_bits,
                                                      uint8_t* __restrict__ out, float* __restrict__ scale_out,
                                                      float* __restrict__ inv_out) {
    const float amax = amax_read(amax_bits);
    const float scale = scale_from_amax(amax, fp8_max<FMT>());
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        if (scale_out) *scale_out = scale;
        *inv_out = 1.0f / scale;
    }
    // 16 elements per thread-iteration: 32 B of bf16 (or 64 B of fp32) in, 16 B out
    const int64_t n16 = n / 16;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x) {
        float f[16];
        if (IS_BF16) {
            const uint4* p = (const uint4*)x + i * 2;
            uint4 a = p[0], b = p[1];
            uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                f[2 * j] = bf16_lo(w[j]);
                f[2 * j + 1] = bf16_hi(w[j]);
            }
        } else {
            const float4* p = (const float4*)x + i * 4;
#pragma unroll
            for (int j = 0; j < 4; j++) {
                float4 v = p[j];
                f[4 * j] = v.x, f[4 * j + 1] = v.y, f[4 * j + 2] = v.z, f[4 * j + 3] = v.w;
            }
        }
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float y0 = fp8_clamp<FMT>(f[4 * j] * scale), y1 = fp8_clamp<FMT>(f[4 * j + 1] * scale);
            float y2 = fp8_clamp<FMT>(f[4 * j + 2] * scale), y3 = fp8_clamp<FMT>(f[4 * j + 3] * scale);
            o[j] = fp8_pack4<FMT, HW_CVT>(y0, y1, y2, y3);
        }
        ((uint4*)out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    if (blockIdx.x == 0) {
        for (int64_t i = n16 * 16 + threadIdx.x; i < n; i += blockDim.x) {
            float v = IS_BF16 ? bf16_to_f32(((const bf16_t*)x)[i]) : ((const float*)x)[i];
            float y = fp8_clamp<FMT>(v * scale);
            out[i] = (uint8_t)(fp8_pack4<FMT, HW_CVT>(y, 0.f, 0.f, 0.f) & 0xffu);
        }
    }
}

__global__ void clear_u32_kernel(uint32_t* p, int n) {
    int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Encode with a caller-given scale (no amax pass): used to check the encoder exhaustively.
template <bool HW_CVT, int FMT>
__global__ void encode_with_scale_kernel(const bf16_t* __restrict__ x, int64_t n, float scale, uint8_t* __restrict__ out) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        float y = fp8_clamp<FMT>(bf16_to_f32(x[i]) * scale);
        out[i] = (uint8_t)(fp8_pack4<FMT, HW_CVT>(y, 0.f, 0.f, 0.f) & 0xffu);
    }
}

static int grid_for(int64_t work_items, int per_block, int max_blocks) {
    int64_t g = (work_items + per_block - 1) / per_block;
    if (g < 1) g = 1;
    if (g > max_blocks) g = max_blocks;
    return (int)g;
}

void nc_clear_u32(uint32_t* p, int n, hipStream_t s) {
    hipLaunchKernelGGL(clear_u32_kernel, dim3((n + 63) / 64), dim3(64), 0, s, p, n);
}

template <int FMT>
static void launch_quantize_fmt(const void* x, int x_dtype, int64_t n, uint8_t* out, float* scale_out, float* inv_out, uint32_t* amax_ws,
                                int encoder, int g1, int g2, hipStream_t s) {
    if (x_dtype == 0) {
        hipLaunchKernelGGL(amax_kernel<true>, dim3(g1), dim3(256), 0, s, x, n, amax_ws);
        if (encoder == 0)
            hipLaunchKernelGGL((convert_kernel<true, true, FMT>), dim3(g2), dim3(256), 0, s, x, n, amax_ws, out, scale_out, inv_out);
        else
            hipLaunchKernelGGL((convert_kernel<true, false, FMT>), dim3(g2), dim3(256), 0, s, x, n, amax_ws, out, scale_out, inv_out);
    } else {
        hipLaunchKernelGGL(amax_kernel<false>, dim3(g1), dim3(256), 0, s, x, n, amax_ws);
        if (encoder == 0)
            hipLaunchKernelGGL((convert_kernel<false, true, FMT>), dim3(g2), dim3(256), 0, s, x, n, amax_ws, out, scale_out, inv_out);
        else
            hipLaunchKernelGGL((convert_kernel<false, false, FMT>), dim3(g2), dim3(256), 0, s, x, n, amax_ws, out, scale_out, inv_out);
    }
}

int nc_launch_quantize(const void* x, int x_dtype, int64_t n, int fmt, uint8_t* out, float* scale_out, float* inv_out,
                       uint32_t* amax_ws, int encoder, hipStream_t s) {
    NC_CHECK_ARG(n >= 0, "fp8_quantize: negative element count");
    NC_CHECK_ARG(inv_out && amax_ws && (n == 0 || (x && out)), "fp8_quantize: null pointer");
    NC_CHECK_ARG(x_dtype == 0 || x_dtype == 1, "fp8_quantize: dtype must be 0 (bf16) or 1 (fp32)");
    NC_CHECK_ARG(fmt == 0 || fmt == 1, "fp8_quantize: format must be 0 (e4m3fn) or 1 (e5m2)");
    NC_CHECK_ARG(((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0, "fp8_quantize: pointers must be 16-byte aligned");
    nc_clear_u32(amax_ws, 1, s);
    NcProfScope prof(2, 3.0 * n, s);
    const int per_vec = x_dtype == 0 ? 8 : 4;
    // at most 1024 blocks x 256 threads, four loads per thread and trip; every block ends with one atomic on the same word
    int g1 = grid_for(n / per_vec, 1024, 1024);
    int g2 = grid_for(n / 16, 256, 4096);
    if (fmt == 0) launch_quantize_fmt<0>(x, x_dtype, n, out, scale_out, inv_out, amax_ws, encoder, g1, g2, s);
    else launch_quantize_fmt<1>(x, x_dtype, n, out, scale_out, inv_out, amax_ws, encoder, g1, g2, s);
    NC_CHECK_LAUNCH("fp8_quantize");
    return 0;
}

// ---------------------------------------------------------------- one launch: amax, grid-wide meeting, convert
// For tensors that fit in the registers of the workgroups the chip can hold at once (up to ~30 M bf16 elements): every thread loads
// its share once and keeps it, the workgroups meet on the tensor's amax, and the payload is converted from registers.  HBM sees the
// algorithmic 3 bytes per element and the three launches (clear, amax, convert) become one.
//
// The meeting needs every workgroup of the grid to be resident, which holds because the grid is sized to half of what the device can
// hold of this kernel alone (hipOccupancyMaxActiveBlocksPerMultiprocessor x CUs): a workgroup that has to wait for a slot taken by
// some other kernel gets it when that kernel ends, and nothing the other kernel does waits for this one.  Two such grids on one GPU
// (of this process or of another) still both fit; more of them at once can hold each other's slots.  The wait is therefore bounded
// (`spin_limit` polls), and a workgroup whose wait runs out does not fail: it works the tensor's amax out by itself, reading the
// whole tensor once more (slow -- a single workgroup streams at tens of GB/s -- and bit-identical, because the maximum does not
// depend on who computes it), converts its share and leaves like every other.  Such workgroups are counted in word 257 of the
// state, which the kernel never reads and never clears: a diagnostic for the host, not a condition.
//
// Ordering.  Everything the workgroups exchange (maxima, arrival counts, the flag, departures) is read and written with device-scope
// atomic operations, which are performed at the device's coherence point, not in an XCD's L2: there is no plain store to make
// visible, hence no release / acquire fence (each of which would write back or invalidate an XCD's whole L2).  Program order
// within the one lane that does them is kept by waiting for the value every read-modify-write returns before the next one is
// issued: the maximum is acknowledged before the arrival is counted, so whoever sees all arrivals sees all maxima.
//
// state: all zero before the first call, left all zero by every call, whichever way its workgroups went (the last workgroup to
// leave clears it; every workgroup leaves exactly once, after it has arrived).  Slot k (k = blockIdx.x % 8) lives on its own
// 128-byte line: word 0 the running maximum, word 1 the arrivals (one address would serialize the grid's atomics at ~6 ns each).
// Line 8: departures, the count of workgroups that ever took the slow way (sticky), slots reported.  Line 9: the flag that the
// last reported slot raises and one lane per workgroup watches.  Line 10, word 0: scratch of the two-pass path.
#define QF_SLOTS 8
#define QF_STRIDE 32
#define QF_DEPART (QF_SLOTS * QF_STRIDE)
#define QF_ERROR (QF_SLOTS * QF_STRIDE + 1)
#define QF_SLOTS_DONE (QF_SLOTS * QF_STRIDE + 2)
#define QF_FLAG ((QF_SLOTS + 1) * QF_STRIDE)
#define QF_SCRATCH ((QF_SLOTS + 2) * QF_STRIDE)
template <int FMT, bool HW_CVT, int G>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(4, 8))) void quantize_fused_kernel(const bf16_t* __restrict__ x, int64_t n16, uint8_t* __restrict__ out,
                                                             float* __restrict__ scale_out, float* __restrict__ inv_out,
                                                             uint32_t* __restrict__ state, uint32_t spin_limit) {
    __shared__ uint32_t red[4];
    __shared__ uint32_t amax_sh, slow_sh;
    const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6;
    // group g of this thread: 16 elements (32 bytes in, 16 bytes out) at group index (blockIdx.x * G + g) * 256 + tid
    uint4 ra[G], rb[G];
    uint32_t m = 0;
#pragma unroll
    for (int g = 0; g < G; g++) {
        int64_t idx = ((int64_t)blockIdx.x * G + g) * 256 + tid;
        idx = idx < n16 ? idx : n16 - 1;                   // a slot past the end re-reads the last group (its maximum is already counted)
        const v4i* p = (const v4i*)x + idx * 2;
        const v4i a = __builtin_nontemporal_load(p), b = __builtin_nontemporal_load(p + 1);
        ra[g] = make_uint4((uint32_t)a[0], (uint32_t)a[1], (uint32_t)a[2], (uint32_t)a[3]);
        rb[g] = make_uint4((uint32_t)b[0], (uint32_t)b[1], (uint32_t)b[2], (uint32_t)b[3]);
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        const uint32_t wd[8] = {ra[g].x, ra[g].y, ra[g].z, ra[g].w, rb[g].x, rb[g].y, rb[g].z, rb[g].w};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t lo = (wd[j] & 0x7fffu) << 16, hi = wd[j] & 0x7fff0000u;
            m = m > lo ? m : lo;
            m = m > hi ? m : hi;
        }
    }
    m = wave_max_u32(m);
    if (lane == 0) red[w] = m;
    __syncthreads();
    if (w == 0) {
        const uint32_t k = blockIdx.x % QF_SLOTS;
        uint32_t* slot = state + k * QF_STRIDE;
        bool gave_up = false;
        if (lane == 0) {
            uint32_t t = red[0];
            for (int i = 1; i < 4; i++) t = t > red[i] ? t : red[i];
            // the maximum first, its acknowledgement awaited (a returning atomic), then the arrival: whoever sees all arrivals sees all maxima
            const uint32_t before = __hip_atomic_fetch_max(slot, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            asm volatile("" ::"v"(before) : "memory");
            const uint32_t in_slot = (gridDim.x - k + QF_SLOTS - 1) / QF_SLOTS;       // workgroups that use this slot
            const uint32_t used = gridDim.x < QF_SLOTS ? gridDim.x : QF_SLOTS;        // slots in use
            // the last arrival of a slot reports the slot; the last slot to be reported raises the flag everyone watches
            if (__hip_atomic_fetch_add(slot + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == in_slot - 1) {
                if (__hip_atomic_fetch_add(state + QF_SLOTS_DONE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == used - 1)
                    __hip_atomic_store(state + QF_FLAG, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            uint32_t spins = 0;
            while (__hip_atomic_load(state + QF_FLAG, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0u) {
                if (++spins > spin_limit) {
                    gave_up = true;
                    break;
                }
                __builtin_amdgcn_s_sleep(8);
            }
        }
        gave_up = __builtin_amdgcn_readfirstlane((int)gave_up) != 0;
        uint32_t am = lane < QF_SLOTS ? __hip_atomic_load(state + lane * QF_STRIDE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0u;
        am = wave_max_u32(am);
        if (lane == 0) {
            amax_sh = am;                                    // (not looked at by a workgroup that gave up: the slots were incomplete)
            slow_sh = gave_up ? 1u : 0u;
            if (gave_up) __hip_atomic_fetch_add(state + QF_ERROR, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            // leave; the last one out puts the state back to zero for the next call (everyone has arrived and read what it needs by
            // now: a workgroup leaves only after its own arrival, with the flag seen or its wait given up)
            const uint32_t gone = __hip_atomic_fetch_add(state + QF_DEPART, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (gone == gridDim.x - 1) {
                for (int i = 0; i < QF_SLOTS; i++) {
                    __hip_atomic_store(state + i * QF_STRIDE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(state + i * QF_STRIDE + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                __hip_atomic_store(state + QF_SLOTS_DONE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(state + QF_FLAG, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_store(state + QF_DEPART, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    __syncthreads();
    if (slow_sh) {
        // the meeting did not complete within this workgroup's wait: the maximum over the whole tensor, by this workgroup alone
        uint32_t mm = 0;
        for (int64_t idx = tid; idx < n16; idx += 256) {
            const uint4 a = ((const uint4*)x)[idx * 2], b = ((const uint4*)x)[idx * 2 + 1];
            const uint32_t wd[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t lo = (wd[j] & 0x7fffu) << 16, hi = wd[j] & 0x7fff0000u;
                mm = mm > lo ? mm : lo;
                mm = mm > hi ? mm : hi;
            }
        }
        mm = wave_max_u32(mm);
        __syncthreads();                                     // red[] was read by wave 0 before the barrier above
        if (lane == 0) red[w] = mm;
        __syncthreads();
        if (tid == 0) {
            uint32_t t = red[0];
            for (int i = 1; i < 4; i++) t = t > red[i] ? t : red[i];
            amax_sh = t;
        }
        __syncthreads();
    }
    const float scale = scale_from_amax(__uint_as_float(amax_sh), fp8_max<FMT>());
    if (blockIdx.x == 0 && tid == 0) {
        if (scale_out) *scale_out = scale;
        *inv_out = 1.0f / scale;
    }
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int64_t idx = ((int64_t)blockIdx.x * G + g) * 256 + tid;
        if (idx >= n16) continue;
        const uint32_t wd[8] = {ra[g].x, ra[g].y, ra[g].z, ra[g].w, rb[g].x, rb[g].y, rb[g].z, rb[g].w};
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float y0 = fp8_clamp<FMT>(bf16_lo(wd[2 * j]) * scale), y1 = fp8_clamp<FMT>(bf16_hi(wd[2 * j]) * scale);
            const float y2 = fp8_clamp<FMT>(bf16_lo(wd[2 * j + 1]) * scale), y3 = fp8_clamp<FMT>(bf16_hi(wd[2 * j + 1]) * scale);
            o[j] = fp8_pack4<FMT, HW_CVT>(y0, y1, y2, y3);
        }
        __builtin_nontemporal_store(v4i{(int)o[0], (int)o[1], (int)o[2], (int)o[3]}, (v4i*)out + idx);
    }
}

// how many workgroups of quantize_fused_kernel<.., G> the current device holds at once (0: unknown, do not use the kernel)
template <int FMT, bool HW_CVT, int G>
static int fused_capacity() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    int cap = cached[dev].load(std::memory_order_relaxed);
    if (cap == 0) {
        int per_cu = 0, cus = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quantize_fused_kernel<FMT, HW_CVT, G>, 256, 0) != hipSuccess) per_cu = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) cus = 0;
        cap = per_cu * cus;
        if (cap <= 0) cap = -1;
        cached[dev].store(cap, std::memory_order_relaxed);
    }
    return cap > 0 ? cap : 0;
}

template <int FMT, bool HW_CVT, int G>
static bool try_fused(const bf16_t* x, int64_t n16, uint8_t* out, float* scale_out, float* inv_out, uint32_t* state, uint32_t spin_limit,
                      hipStream_t s) {
    const int64_t blocks = (n16 + 256 * (int64_t)G - 1) / (256 * (int64_t)G);
    // half of the capacity: two such grids on one GPU at the same time still both fit (more than that can hold each other's slots
    // until the bounded wait runs out and the workgroups take the slow way)
    if (blocks > (int64_t)fused_capacity<FMT, HW_CVT, G>() / 2) return false;
    hipLaunchKernelGGL((quantize_fused_kernel<FMT, HW_CVT, G>), dim3((unsigned)blocks), dim3(256), 0, s, x, n16, out, scale_out, inv_out, state,
                       spin_limit);
    return true;
}

template <int FMT, bool HW_CVT>
static bool try_fused_any(const bf16_t* x, int64_t n16, uint8_t* out, float* scale_out, float* inv_out, uint32_t* state, uint32_t lim,
                          hipStream_t s) {
    // The largest share per thread that still leaves a workgroup for every other CU: few workgroups keep the meeting cheap (its atomics and
    // its pollers share a handful of memory lines), long shares keep many loads in flight per thread.
    const int64_t per_wg = 128;          // (half of the CUs at least)
    if (n16 >= 8 * per_wg * 256 && try_fused<FMT, HW_CVT, 8>(x, n16, out, scale_out, inv_out, state, lim, s)) return true;
    if (n16 >= 4 * per_wg * 256 && try_fused<FMT, HW_CVT, 4>(x, n16, out, scale_out, inv_out, state, lim, s)) return true;
    if (n16 >= 2 * per_wg * 256 && try_fused<FMT, HW_CVT, 2>(x, n16, out, scale_out, inv_out, state, lim, s)) return true;
    return try_fused<FMT, HW_CVT, 1>(x, n16, out, scale_out, inv_out, state, lim, s) || try_fused<FMT, HW_CVT, 2>(x, n16, out, scale_out, inv_out, state, lim, s) ||
           try_fused<FMT, HW_CVT, 4>(x, n16, out, scale_out, inv_out, state, lim, s) || try_fused<FMT, HW_CVT, 8>(x, n16, out, scale_out, inv_out, state, lim, s);
}

// state: NC_QUANTIZE_STATE_BYTES (1 KB + 16).  Tensors the one-launch kernel does not take (fp32 input, an element count that is
// not a multiple of 16, more elements than fit on the chip) go through the two passes, with the state's last word as their scratch.
// spin_limit: polls of the meeting's flag (a few hundred ns each) before a workgroup stops waiting and takes the slow way;
// NC_QUANTIZE_DEFAULT_SPINS in ordinary use, a tiny value from the test that drives the slow way.
int nc_launch_quantize_fused(const void* x, int x_dtype, int64_t n, int fmt, uint8_t* out, float* scale_out, float* inv_out,
                             uint32_t* state, int encoder, hipStream_t s, uint32_t spin_limit) {
    NC_CHECK_ARG(n >= 0, "fp8_quantize: negative element count");
    NC_CHECK_ARG(inv_out && state && (n == 0 || (x && out)), "fp8_quantize: null pointer");
    NC_CHECK_ARG(x_dtype == 0 || x_dtype == 1, "fp8_quantize: dtype must be 0 (bf16) or 1 (fp32)");
    NC_CHECK_ARG(fmt == 0 || fmt == 1, "fp8_quantize: format must be 0 (e4m3fn) or 1 (e5m2)");
    NC_CHECK_ARG(((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)state & 127) == 0,
                 "fp8_quantize: pointers must be 16-byte aligned (the state 128-byte aligned)");
    if (x_dtype == 0 && n >= 16 && n % 16 == 0) {
        NcProfScope prof(2, 3.0 * n, s);
        const bf16_t* xb = (const bf16_t*)x;
        bool done;
        if (fmt == 0) done = encoder == 0 ? try_fused_any<0, true>(xb, n / 16, out, scale_out, inv_out, state, spin_limit, s)
                                          : try_fused_any<0, false>(xb, n / 16, out, scale_out, inv_out, state, spin_limit, s);
        else done = encoder == 0 ? try_fused_any<1, true>(xb, n / 16, out, scale_out, inv_out, state, spin_limit, s)
                                 : try_fused_any<1, false>(xb, n / 16, out, scale_out, inv_out, state, spin_limit, s);
        if (done) {
            NC_CHECK_LAUNCH("fp8_quantize");
            return 0;
        }
    }
    return nc_launch_quantize(x, x_dtype, n, fmt, out, scale_out, inv_out, state + QF_SCRATCH, encoder, s);
}

// Convert only, with amax already reduced into amax_ws by a producer kernel.
int nc_launch_convert_only(const void* x, int64_t n, uint8_t* out, float* inv_out, const uint32_t* amax_ws, hipStream_t s) {
    NcProfScope prof(2, 3.0 * n, s);
    int g2 = grid_for(n / 16, 256, 4096);
    hipLaunchKernelGGL((convert_kernel<true, true>), dim3(g2), dim3(256), 0, s, x, n, amax_ws, out, (float*)nullptr, inv_out);
    NC_CHECK_LAUNCH("fp8_convert");
    return 0;
}

int nc_launch_encode_with_scale(const bf16_t* x, int64_t n, float scale, int fmt, uint8_t* out, int encoder, hipStream_t s) {
    NC_CHECK_ARG(x && out && n >= 0, "fp8_encode: bad arguments");
    NC_CHECK_ARG(fmt == 0 || fmt == 1, "fp8_encode: format must be 0 (e4m3fn) or 1 (e5m2)");
    int g = (int)((n + 255) / 256);
    if (g == 0) return 0;
    if (fmt == 0) {
        if (encoder == 0) hipLaunchKernelGGL((encode_with_scale_kernel<true, 0>), dim3(g), dim3(256), 0, s, x, n, scale, out);
        else hipLaunchKernelGGL((encode_with_scale_kernel<false, 0>), dim3(g), dim3(256), 0, s, x, n, scale, out);
    } else {
        if (encoder == 0) hipLaunchKernelGGL((encode_with_scale_kernel<true, 1>), dim3(g), dim3(256), 0, s, x, n, scale, out);
        else hipLaunchKernelGGL((encode_with_scale_kernel<false, 1>), dim3(g), dim3(256), 0, s, x, n, scale, out);
    }
    NC_CHECK_LAUNCH("fp8_encode");
    return 0;
}

// ---------------------------------------------------------------- byte-matrix transpose
// dst[c][r] = src[r][c] for an fp8 payload: the memory rearrangement behind _to_col_major and .t().contiguous() at
// nanochat/fp8.py:110-118,169,181-182 (the backward GEMMs need the reduction index contiguous in both operands).
// 128x128 tiles: 16-byte global accesses on both sides (whole 128-byte row segments), 4x4 byte blocks transposed in
// registers with v_perm_b32 between two LDS copies of the tile.
#define TP_PITCH 144
__global__ __launch_bounds__(256) void transpose_u8_kernel(const uint8_t* __restrict__ src, int R, int C, uint8_t* __restrict__ dst) {
    __shared__ __align__(16) uint8_t ta[128 * TP_PITCH], tb[128 * TP_PITCH];
    const int r0 = blockIdx.y * 128, c0 = blockIdx.x * 128, t = threadIdx.x;
    const int lrow = t >> 3, lc16 = (t & 7) * 16;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = lrow + 32 * i;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (r0 + row < R && c0 + lc16 < C) v = *(const uint4*)(src + (size_t)(r0 + row) * C + c0 + lc16);
        *(uint4*)(ta + row * TP_PITCH + lc16) = v;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int blk = t + 256 * i, rb = blk >> 5, cb = blk & 31;      // 4x4 block: rows 4 rb.., columns 4 cb..
        uint32_t d[4];
#pragma unroll
        for (int k = 0; k < 4; k++) d[k] = *(const uint32_t*)(ta + (4 * rb + k) * TP_PITCH + 4 * cb);
        const uint32_t t0 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400), t1 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602);
        const uint32_t u0 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400), u1 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602);
        const uint32_t o[4] = {__builtin_amdgcn_perm(u0, t0, 0x05040100), __builtin_amdgcn_perm(u0, t0, 0x07060302),
                               __builtin_amdgcn_perm(u1, t1, 0x05040100), __builtin_amdgcn_perm(u1, t1, 0x07060302)};
#pragma unroll
        for (int k = 0; k < 4; k++) *(uint32_t*)(tb + (4 * cb + k) * TP_PITCH + 4 * rb) = o[k];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = lrow + 32 * i;          // a column of src
        if (c0 + row < C && r0 + lc16 < R)
            *(uint4*)(dst + (size_t)(c0 + row) * R + r0 + lc16) = *(const uint4*)(tb + row * TP_PITCH + lc16);
    }
}

// ---------------------------------------------------------------- convert + transpose in one pass
// out[r][c] = fp8(x[r][c]) and out_t[c][r] = the same byte, from one read of x (amax already reduced into amax_bits): what the
// backward GEMMs of nanochat/fp8.py:156-192 need of the output gradient (both grad_output in e5m2 and its transpose) and, saved by
// the forward, of the input (its transpose for grad_weight).  128 x 128 tiles: every thread converts eight 16-byte pieces of bf16
// (coalesced 256-byte row segments), stores the eight payload bytes row-major straight from registers (16 lanes = one 128-byte
// line) and into an LDS copy of the tile, which then goes through the 4 x 4 byte transposes of transpose_u8_kernel.
template <int FMT>
__global__ __launch_bounds__(256) void convert_transpose_kernel(const bf16_t* __restrict__ x, int R, int C, const uint32_t* __restrict__ amax_bits,
                                                                uint8_t* __restrict__ out, uint8_t* __restrict__ out_t,
                                                                float* __restrict__ scale_out, float* __restrict__ inv_out) {
    __shared__ __align__(16) uint8_t ta[128 * TP_PITCH], tb[128 * TP_PITCH];
    const int r0 = blockIdx.y * 128, c0 = blockIdx.x * 128, t = threadIdx.x;
    uint4 in[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = t + 256 * i, row = q >> 4, c8 = (q & 15) * 8;
        in[i] = make_uint4(0, 0, 0, 0);
        if (r0 + row < R && c0 + c8 < C) in[i] = *(const uint4*)(x + (size_t)(r0 + row) * C + c0 + c8);
    }
    const float scale = scale_from_amax(amax_read(amax_bits), fp8_max<FMT>());
    if (blockIdx.x == 0 && blockIdx.y == 0 && t == 0) {
        if (scale_out) *scale_out = scale;
        *inv_out = 1.0f / scale;
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int q = t + 256 * i, row = q >> 4, c8 = (q & 15) * 8;
        const uint32_t w[4] = {in[i].x, in[i].y, in[i].z, in[i].w};
        uint32_t o[2];
#pragma unroll
        for (int j = 0; j < 2; j++)
            o[j] = fp8_pack4<FMT, true>(fp8_clamp<FMT>(bf16_lo(w[2 * j]) * scale), fp8_clamp<FMT>(bf16_hi(w[2 * j]) * scale),
                                        fp8_clamp<FMT>(bf16_lo(w[2 * j + 1]) * scale), fp8_clamp<FMT>(bf16_hi(w[2 * j + 1]) * scale));
        *(uint2*)(ta + row * TP_PITCH + c8) = make_uint2(o[0], o[1]);
        if (r0 + row < R && c0 + c8 < C) *(uint2*)(out + (size_t)(r0 + row) * C + c0 + c8) = make_uint2(o[0], o[1]);
    }
    __syncthreads();
    const int lrow = t >> 3, lc16 = (t & 7) * 16;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int blk = t + 256 * i, rb = blk >> 5, cb = blk & 31;      // 4x4 block: rows 4 rb.., columns 4 cb..
        uint32_t d[4];
#pragma unroll
        for (int k = 0; k < 4; k++) d[k] = *(const uint32_t*)(ta + (4 * rb + k) * TP_PITCH + 4 * cb);
        const uint32_t t0 = __builtin_amdgcn_perm(d[1], d[0], 0x05010400), t1 = __builtin_amdgcn_perm(d[1], d[0], 0x07030602);
        const uint32_t u0 = __builtin_amdgcn_perm(d[3], d[2], 0x05010400), u1 = __builtin_amdgcn_perm(d[3], d[2], 0x07030602);
        const uint32_t o[4] = {__builtin_amdgcn_perm(u0, t0, 0x05040100), __builtin_amdgcn_perm(u0, t0, 0x07060302),
                               __builtin_amdgcn_perm(u1, t1, 0x05040100), __builtin_amdgcn_perm(u1, t1, 0x07060302)};
#pragma unroll
        for (int k = 0; k < 4; k++) *(uint32_t*)(tb + (4 * cb + k) * TP_PITCH + 4 * rb) = o[k];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int row = lrow + 32 * i;          // a column of x
        if (c0 + row < C && r0 + lc16 < R)
            *(uint4*)(out_t + (size_t)(c0 + row) * R + r0 + lc16) = *(const uint4*)(tb + row * TP_PITCH + lc16);
    }
}

int nc_launch_quantize_transposed(const bf16_t* x, int R, int C, int fmt, uint8_t* out, uint8_t* out_t, float* scale_out, float* inv_out,
                                  uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(R >= 0 && C >= 0, "fp8_quantize_transposed: negative shape");
    NC_CHECK_ARG(inv_out && amax_ws, "fp8_quantize_transposed: null pointer");
    NC_CHECK_ARG(fmt == 0 || fmt == 1, "fp8_quantize_transposed: format must be 0 (e4m3fn) or 1 (e5m2)");
    if (R == 0 || C == 0) return 0;
    NC_CHECK_ARG(x && out && out_t, "fp8_quantize_transposed: null pointer");
    NC_CHECK_ARG(R % 16 == 0 && C % 16 == 0, "fp8_quantize_transposed: rows=%d and cols=%d must be multiples of 16", R, C);
    NC_CHECK_ARG((((uintptr_t)x | (uintptr_t)out | (uintptr_t)out_t) & 15) == 0, "fp8_quantize_transposed: pointers must be 16-byte aligned");
    const int64_t n = (int64_t)R * C;
    nc_clear_u32(amax_ws, 1, s);
    NcProfScope prof(2, 4.0 * n, s);             // 2 bytes read + 2 x 1 byte written per element
    hipLaunchKernelGGL(amax_kernel<true>, dim3(grid_for(n / 8, 1024, 1024)), dim3(256), 0, s, (const void*)x, n, amax_ws);
    const dim3 grid((C + 127) / 128, (R + 127) / 128);
    if (fmt == 0) hipLaunchKernelGGL(convert_transpose_kernel<0>, grid, dim3(256), 0, s, x, R, C, amax_ws, out, out_t, scale_out, inv_out);
    else hipLaunchKernelGGL(convert_transpose_kernel<1>, grid, dim3(256), 0, s, x, R, C, amax_ws, out, out_t, scale_out, inv_out);
    NC_CHECK_LAUNCH("fp8_quantize_transposed");
    return 0;
}

int nc_launch_transpose_u8(const uint8_t* src, int R, int C, uint8_t* dst, hipStream_t s) {
    NC_CHECK_ARG(R >= 0 && C >= 0, "fp8_transpose: negative shape");
    if (R == 0 || C == 0) return 0;
    NC_CHECK_ARG(src && dst, "fp8_transpose: null pointer");
    NC_CHECK_ARG(R % 16 == 0 && C % 16 == 0, "fp8_transpose: rows=%d and cols=%d must be multiples of 16", R, C);
    NC_CHECK_ARG(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, "fp8_transpose: pointers must be 16-byte aligned");
    hipLaunchKernelGGL(transpose_u8_kernel, dim3((C + 127) / 128, (R + 127) / 128), dim3(256), 0, s, src, R, C, dst);
    NC_CHECK_LAUNCH("fp8_transpose");
    return 0;
}

