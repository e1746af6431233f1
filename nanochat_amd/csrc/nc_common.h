// Shared device/host helpers for the gfx950 kernels: bf16 and e4m3 conversion, wave64
// reductions over DPP, and the error channel of the C ABI.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define NC_WAVE 64

typedef uint16_t bf16_t;   // raw bfloat16 bits
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------- error channel (host)
void nc_set_error(const char* fmt, ...);
#define NC_FAIL(code, ...)        \
    do {                          \
        nc_set_error(__VA_ARGS__); \
        return (code);            \
    } while (0)
#define NC_CHECK_ARG(cond, ...)            \
    do {                                   \
        if (!(cond)) NC_FAIL(-1, __VA_ARGS__); \
    } while (0)
#define NC_CHECK_LAUNCH(name)                                                        \
    do {                                                                             \
        hipError_t e__ = hipGetLastError();                                          \
        if (e__ != hipSuccess) NC_FAIL(-2, "%s: launch failed: %s", name, hipGetErrorString(e__)); \
    } while (0)

// ---------------------------------------------------------------- bf16
__device__ __forceinline__ float bf16_to_f32(bf16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

// fp32 -> bf16, round to nearest even (NaN stays NaN): gfx950's own convert (v_cvt_pk_bf16_f32), one instruction where the integer form (NaN test,
// rounding increment, shift) takes six; the row kernels round after every elementary operation, so this is most of their arithmetic
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }
// value of f after rounding to bf16, as fp32 (one rounding site of a bf16 eager op)
__device__ __forceinline__ float rbf(float f) { return bf16_to_f32(f32_to_bf16(f)); }
// two fp32 -> packed bf16 pair (one convert instruction), low half = first value
typedef __bf16 nc_bf16x2 __attribute__((ext_vector_type(2)));
typedef float nc_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    const nc_f32x2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, nc_bf16x2));
}
__device__ __forceinline__ uint32_t pack_bf16_hw(float lo, float hi) { return pack_bf16(lo, hi); }

// ---------------------------------------------------------------- e4m3fn (OCP) encode
// |y| must already be clamped to <= 448.  Round to nearest even, subnormals down to 2^-9.
__device__ __forceinline__ uint32_t e4m3_encode_sw(float y) {
    uint32_t u = __float_as_uint(y);
    uint32_t sign = (u >> 24) & 0x80u;
    u &= 0x7fffffffu;
    uint32_t out;
    if (u >= 0x3c800000u) {                      // >= 2^-6: normal in e4m3
        u += 0x7ffffu + ((u >> 20) & 1u);        // RNE at mantissa bit 20
        out = (u >> 20) - ((127u - 7u) << 3);
    } else {                                     // subnormal: multiples of 2^-9
        float m = __uint_as_float(u) * 512.0f;   // exact
        out = (uint32_t)__builtin_rintf(m);      // 0..8, ties to even; 8 == 0x08 == 2^-6
    }
    return sign | out;
}

// four fp32 (already scaled and clamped) -> four packed e4m3 bytes, hardware convert
__device__ __forceinline__ uint32_t e4m3_pack4_hw(float a, float b, float c, float d) {
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
    return (uint32_t)r;
}
__device__ __forceinline__ uint32_t e4m3_pack4_sw(float a, float b, float c, float d) {
    return e4m3_encode_sw(a) | (e4m3_encode_sw(b) << 8) | (e4m3_encode_sw(c) << 16) | (e4m3_encode_sw(d) << 24);
}
__device__ __forceinline__ float clamp448(float y) { return fminf(fmaxf(y, -448.0f), 448.0f); }

// ---------------------------------------------------------------- e5m2 (OCP) encode: the gradient format of nanochat/fp8.py:165
// |y| must already be clamped to <= 57344.  Round to nearest even, subnormals down to 2^-16.  e5m2 is the top byte of fp16.
__device__ __forceinline__ uint32_t e5m2_encode_sw(float y) {
    uint32_t u = __float_as_uint(y);
    uint32_t sign = (u >> 24) & 0x80u;
    u &= 0x7fffffffu;
    uint32_t out;
    if (u >= 0x38800000u) {                      // >= 2^-14: normal in e5m2
        u += 0xfffffu + ((u >> 21) & 1u);        // RNE at mantissa bit 21
        out = (u >> 21) - ((127u - 15u) << 2);
    } else {                                     // subnormal: multiples of 2^-16
        float m = __uint_as_float(u) * 65536.0f; // exact
        out = (uint32_t)__builtin_rintf(m);      // 0..4, ties to even; 4 == 0x04 == 2^-14
    }
    return sign | out;
}
__device__ __forceinline__ uint32_t e5m2_pack4_hw(float a, float b, float c, float d) {
    int r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
    return (uint32_t)r;
}
__device__ __forceinline__ uint32_t e5m2_pack4_sw(float a, float b, float c, float d) {
    return e5m2_encode_sw(a) | (e5m2_encode_sw(b) << 8) | (e5m2_encode_sw(c) << 16) | (e5m2_encode_sw(d) << 24);
}
// FMT 0 = e4m3fn (max 448), 1 = e5m2 (max 57344)
template <int FMT> __device__ __forceinline__ float fp8_max() { return FMT == 0 ? 448.0f : 57344.0f; }
template <int FMT> __device__ __forceinline__ float fp8_clamp(float y) { return fminf(fmaxf(y, -fp8_max<FMT>()), fp8_max<FMT>()); }
template <int FMT, bool HW> __device__ __forceinline__ uint32_t fp8_pack4(float a, float b, float c, float d) {
    if (FMT == 0) return HW ? e4m3_pack4_hw(a, b, c, d) : e4m3_pack4_sw(a, b, c, d);
    return HW ? e5m2_pack4_hw(a, b, c, d) : e5m2_pack4_sw(a, b, c, d);
}

// scale = fp32(448 / max(fp64(amax), 1e-12)) -- the divide is done in fp64 like the reference
__device__ __forceinline__ float scale_from_amax(float amax, double fmax = 448.0) {
    double d = (double)amax;
    if (d < 1e-12) d = 1e-12;
    return (float)(fmax / d);
}

// 16-byte load of data that is read once and is larger than the caches (KV cache, weights at decode time): a
// non-temporal load is not kept on its way in; a pure streaming read measures ~15% more HBM bandwidth with it.
__device__ __forceinline__ uint4 nt_load16(const void* p) {
    const v4i r = __builtin_nontemporal_load((const v4i*)p);
    return make_uint4((uint32_t)r[0], (uint32_t)r[1], (uint32_t)r[2], (uint32_t)r[3]);
}

// ---------------------------------------------------------------- wave64 reductions
// DPP row_ror within rows of 16 lanes: all 16 lanes end with the row total.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0x128>(v);   // row_ror:8
    v += dpp_f32<0x124>(v);   // row_ror:4
    v += dpp_f32<0x122>(v);   // row_ror:2
    v += dpp_f32<0x121>(v);   // row_ror:1
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += __shfl_xor(v, 16);
    v += __shfl_xor(v, 32);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
// Running maximum of magnitudes that a NaN survives, as it survives the reference's x.abs().max() (nanochat/fp8.py:92): magnitudes are
// compared as unsigned bit patterns, which order like the values for non-negative floats and put every NaN above infinity.  (fmaxf
// returns the other operand when one is NaN, which would hide a NaN activation from the scale of the next FP8 linear.)
__device__ __forceinline__ float amax_join(float a, float b) {            // both already magnitudes (sign bit clear)
    const uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
    return __uint_as_float(ua > ub ? ua : ub);
}
__device__ __forceinline__ float amax_fold(float am, float x) { return amax_join(am, __uint_as_float(__float_as_uint(x) & 0x7fffffffu)); }
// relu that keeps a NaN, as torch.relu does (fmaxf(x, 0) would turn it into 0)
__device__ __forceinline__ float relu_keep_nan(float x) { return x < 0.f ? 0.f : x; }
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        uint32_t t = (uint32_t)__shfl_xor((int)v, o);
        v = v > t ? v : t;
    }
    return v;
}

__device__ __forceinline__ float wave_amax(float am) { return __uint_as_float(wave_max_u32(__float_as_uint(am))); }

// ---------------------------------------------------------------- cross-workgroup hand-off without cache flushes
// Split results travel between workgroups through device-scope relaxed atomic accesses: such stores are
// written through to the device coherence point and such loads are served from it, so no L2 write-back /
// invalidate (what a device-scope fence costs on a multi-XCD part) is needed.  Ordering against the
// arrival counter comes from waiting for the stores to complete before the counter is bumped.
__device__ __forceinline__ void coherent_store_f4(float* p, float a, float b, float c, float d) {
    unsigned long long lo = ((unsigned long long)__float_as_uint(b) << 32) | __float_as_uint(a);
    unsigned long long hi = ((unsigned long long)__float_as_uint(d) << 32) | __float_as_uint(c);
    __hip_atomic_store((unsigned long long*)p, lo, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store((unsigned long long*)p + 1, hi, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void coherent_load_f4(const float* p, float& a, float& b, float& c, float& d) {
    unsigned long long lo = __hip_atomic_load((const unsigned long long*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned long long hi = __hip_atomic_load((const unsigned long long*)p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    a = __uint_as_float((uint32_t)lo), b = __uint_as_float((uint32_t)(lo >> 32));
    c = __uint_as_float((uint32_t)hi), d = __uint_as_float((uint32_t)(hi >> 32));
}
__device__ __forceinline__ void coherent_store_f1(float* p, float a) {
    __hip_atomic_store((uint32_t*)p, __float_as_uint(a), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float coherent_load_f1(const float* p) {
    return __uint_as_float(__hip_atomic_load((const uint32_t*)p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT));
}
// All of this workgroup's coherent stores are complete when this returns on every thread (call from all threads);
// returns true in every thread of the workgroup that arrived last at `counter` (of `expected` arrivals).
__device__ __forceinline__ bool arrive_and_check_last(uint32_t* counter, uint32_t expected, int* flag_lds) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);       // vmcnt(0) expcnt(0) lgkmcnt(0): every store issued above has been acknowledged
    __syncthreads();
    if (threadIdx.x == 0) {
        const uint32_t old = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag_lds = (old == expected - 1u);
    }
    __syncthreads();
    const bool last = *flag_lds != 0;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    return last;
}

// A kernel argument named here is fetched in the entry block.  The compiler otherwise fetches arguments where they are first used,
// behind whatever branch that is, and a kernel whose body is a few microseconds long then makes several dependent trips to the
// argument segment before its first data load.
#define NC_ARG_NOW(a) asm volatile("" ::"s"(a))

// ---------------------------------------------------------------- amax words
// The tensorwise amax of an activation is max-reduced by its producer kernel into a device word (fp32 bit patterns
// of non-negative values order like integers) and read by the FP8 linear that quantizes the activation.  Atomics on
// one address serialize at the device coherence point (~6 ns each across XCDs: 832 workgroups ending together cost
// ~3.5 us), so the forward pass gives every site NC_AMAX_SLOTS words on separate 128-byte lines: a producer workgroup
// publishes into the slot its block index selects, a consumer takes the max over the slots.  A pointer to such a
// site carries tag bit 0 (nc_amax_slotted); an untagged pointer is a single word (the stand-alone entry points).
// Only amax_read / amax_publish may look through these pointers.
#define NC_AMAX_SLOTS 8
#define NC_AMAX_STRIDE 32      // words between slots
static inline uint32_t* nc_amax_slotted(uint32_t* site) { return (uint32_t*)((uintptr_t)site | 1u); }

__device__ __forceinline__ float amax_read(const uint32_t* h) {
    const uint32_t* p = (const uint32_t*)((uintptr_t)h & ~(uintptr_t)3);
    uint32_t m = p[0];
    if ((uintptr_t)h & 1u) {
#pragma unroll
        for (int i = 1; i < NC_AMAX_SLOTS; i++) {
            const uint32_t v = p[i * NC_AMAX_STRIDE];
            m = v > m ? v : m;
        }
    }
    return __uint_as_float(m);
}
// The same read split in two, for kernels that put all their loads ahead of their first wait: every lane issues one load (lane i < 8
// takes slot i of a slotted site, every other lane the first word), no branch in between; the value is the maximum over lanes 0..7.
__device__ __forceinline__ uint32_t amax_load_lane(const uint32_t* h) {
    const uint32_t* p = (const uint32_t*)((uintptr_t)h & ~(uintptr_t)3);
    const int lane = threadIdx.x & 63;
    return p[(((uintptr_t)h & 1u) && lane < NC_AMAX_SLOTS) ? lane * NC_AMAX_STRIDE : 0];
}
// (lane reads that do not depend on which lanes are active, so this may sit inside divergent code as long as the load did not)
__device__ __forceinline__ float amax_from_lanes(uint32_t loaded) {
    uint32_t m = 0u;
#pragma unroll
    for (int i = 0; i < NC_AMAX_SLOTS; i++) {
        const uint32_t v = (uint32_t)__builtin_amdgcn_readlane((int)loaded, i);
        m = v > m ? v : m;
    }
    return __uint_as_float(m);
}
// And through the scalar cache, for a kernel whose vector loads must not queue behind it: scalar loads have a counter of their own,
// so the words can be asked for first and looked at last without the compiler having to count vector loads in between.
struct AmaxWords { uint32_t w[NC_AMAX_SLOTS]; };
__device__ __forceinline__ AmaxWords amax_load_scalar(const uint32_t* h) {
    // (the constant address space is what makes these scalar loads: a generic pointer built from an integer gets flat loads, which
    // count against both counters and force the vector loads around them to drain)
    typedef const __attribute__((address_space(4))) uint32_t* cptr;
    cptr p = (cptr)((uintptr_t)h & ~(uintptr_t)3);
    const int stride = ((uintptr_t)h & 1u) ? NC_AMAX_STRIDE : 0;
    AmaxWords a;
#pragma unroll
    for (int i = 0; i < NC_AMAX_SLOTS; i++) a.w[i] = p[i * stride];
    return a;
}
__device__ __forceinline__ float amax_from_words(AmaxWords a) {
    uint32_t m = 0u;
#pragma unroll
    for (int i = 0; i < NC_AMAX_SLOTS; i++) {
        m = a.w[i] > m ? a.w[i] : m;
    }
    return __uint_as_float(m);
}
// One call per workgroup.  The atomic is skipped when the word already holds at least the value.
__device__ __forceinline__ void amax_publish(uint32_t* h, float am) {
    const uint32_t bits = __float_as_uint(am);
    if (bits == 0u || (bits >> 31)) return;
    uint32_t* p = (uint32_t*)((uintptr_t)h & ~(uintptr_t)3);
    if ((uintptr_t)h & 1u) p += ((blockIdx.x + 3u * blockIdx.y + 5u * blockIdx.z) % NC_AMAX_SLOTS) * NC_AMAX_STRIDE;
    // with hundreds of workgroups per slot the atomics queue up behind each other and a look first pays; with a few, the look is
    // a round trip to memory in front of an atomic that nobody waits for
    if (gridDim.x * gridDim.y * gridDim.z > 16 * NC_AMAX_SLOTS && __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= bits) return;
    atomicMax(p, bits);
}

// block-wide sum for blockDim.x == 64 * NW, result broadcast to every thread
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red /* >= NW floats of LDS */) {
    v = wave_sum(v);
    if (NW == 1) return v;
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < NW; i++) t += red[i];
    return t;
}
