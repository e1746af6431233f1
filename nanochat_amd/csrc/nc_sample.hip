// Logit softcap and next-token selection.
//   softcap:  logits = softcap * tanh(float(bf16 lm_head output) / softcap)      nanochat/gpt.py:511-515
//   sample:   temperature == 0 -> argmax (first index on ties);
//             top-k -> the k largest logits in descending order, / temperature, softmax over k,
//             then the multinomial draw written as its definition argmax_j(p_j / e_j), e_j ~ Exp(1)
//             supplied by the caller (drawn from the torch generator)            nanochat/engine.py:140-156
//             no top-k -> softmax over the whole vocabulary and the same draw.
// One workgroup per batch row; a row of 32768 fp32 logits is 128 KB and is re-read from L2 by the
// radix-select passes.  Bandwidth bound: B * V * 4 bytes from HBM once.
#include "nc_common.h"
#include "nc_kernels.h"

#define SAMPLE_THREADS 256
#define MAX_TOP_K 4096          // the larger of the two instantiations below (256 and 4096 candidates in LDS)

__global__ __launch_bounds__(256) void softcap_kernel(const bf16_t* __restrict__ raw, float* __restrict__ out, int64_t n, float softcap) {
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x)
        out[i] = softcap * tanhf(bf16_to_f32(raw[i]) / softcap);
}

// order-preserving map float -> uint32 (larger float <=> larger key)
__device__ __forceinline__ uint32_t fkey(float f) {
    uint32_t u = __float_as_uint(f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float fkey_inv(uint32_t k) {
    uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
    return __uint_as_float(u);
}

// (value desc, index asc) argmax across the block; returns the winner to every thread
__device__ __forceinline__ void block_argmax(float& v, int& i, float* sval, int* sidx) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o);
        const int oi = __shfl_xor(i, o);
        if (ov > v || (ov == v && oi < i)) v = ov, i = oi;
    }
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) sval[w] = v, sidx[w] = i;
    __syncthreads();
    v = sval[0], i = sidx[0];
    for (int k = 1; k < SAMPLE_THREADS / 64; k++)
        if (sval[k] > v || (sval[k] == v && sidx[k] < i)) v = sval[k], i = sidx[k];
}

// f(value, index) over one row of logits, 16-byte loads with NF in flight per thread when the row is aligned (a row of 32768
// logits is 32 such loads per thread: with four in flight the scan is eight trips to memory, with sixteen it is two)
template <int NF = 4, typename F>
__device__ __forceinline__ void scan_row(const float* __restrict__ lr, int V, int tid, F f) {
    int done = 0;
    if (((uintptr_t)lr & 15) == 0) {
        const int nv = V >> 2;
        const float4* p = (const float4*)lr;
        int i = tid;
        for (; i + (NF - 1) * SAMPLE_THREADS < nv; i += NF * SAMPLE_THREADS) {
            float4 r[NF];
#pragma unroll
            for (int u = 0; u < NF; u++) r[u] = p[i + u * SAMPLE_THREADS];
#pragma unroll
            for (int u = 0; u < NF; u++) {
                const int b = 4 * (i + u * SAMPLE_THREADS);
                f(r[u].x, b), f(r[u].y, b + 1), f(r[u].z, b + 2), f(r[u].w, b + 3);
            }
        }
        for (; i < nv; i += SAMPLE_THREADS) {
            const float4 r = p[i];
            f(r.x, 4 * i), f(r.y, 4 * i + 1), f(r.z, 4 * i + 2), f(r.w, 4 * i + 3);
        }
        done = nv * 4;
    }
    for (int i = done + tid; i < V; i += SAMPLE_THREADS) f(lr[i], i);
}

template <int KMAX>
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(const float* __restrict__ logits, int V, int ld, float temperature,
                                                                int top_k, const float* __restrict__ noise, int64_t* __restrict__ out_ids) {
    __shared__ float sval[4];
    __shared__ int sidx[4];
    __shared__ uint32_t hist[256];
    __shared__ uint32_t sel_prefix, sel_need;
    __shared__ unsigned long long cand[KMAX];         // (key << 32) | ~index : sorts by value desc, index asc
    __shared__ uint32_t cand_count;
    __shared__ uint32_t scan[SAMPLE_THREADS];
    __shared__ float probs[KMAX];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* lr = logits + (size_t)row * ld;

    if (temperature == 0.0f) {
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        scan_row<16>(lr, V, tid, [&](float v, int i) {
            if (v > bv || (v == bv && i < bi)) bv = v, bi = i;      // NaN never wins; an all-NaN row yields index 0 below
        });
        block_argmax(bv, bi, sval, sidx);
        if (tid == 0) out_ids[row] = (bi == 0x7fffffff) ? 0 : bi;
        return;
    }

    if (top_k <= 0 || top_k >= V) {
        // full-vocabulary softmax: argmax_i exp((l_i - max)/T) / e_i  ==  argmax_i (l_i/T - max/T - log e_i)
        float mx = -INFINITY;
        int dummy = 0;
        scan_row(lr, V, tid, [&](float v, int) { mx = fmaxf(mx, v / temperature); });
        block_argmax(mx, dummy, sval, sidx);
        float bv = -INFINITY;
        int bi = 0x7fffffff;
        for (int i = tid; i < V; i += SAMPLE_THREADS) {
            const float p = expf(lr[i] / temperature - mx) / noise[(size_t)row * V + i];
            if (p > bv || (p == bv && i < bi)) bv = p, bi = i;
        }
        block_argmax(bv, bi, sval, sidx);
        if (tid == 0) out_ids[row] = (bi == 0x7fffffff) ? 0 : bi;
        return;
    }

    // ---- radix select of the k-th largest key, 8 bits per pass from the top
    const uint32_t k = (uint32_t)top_k;
    if (tid == 0) sel_prefix = 0, sel_need = k, cand_count = 0;
    for (int pass = 0; pass < 4; pass++) {
        const int shift = 24 - 8 * pass;
        hist[tid] = 0;
        __syncthreads();
        const uint32_t prefix = sel_prefix;
        const uint32_t himask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
        scan_row(lr, V, tid, [&](float v, int) {
            const uint32_t key = fkey(v);
            if ((key & himask) == prefix) atomicAdd(&hist[(key >> shift) & 0xff], 1u);
        });
        __syncthreads();
        if (tid == 0) {
            uint32_t need = sel_need, bin = 255;
            for (;; bin--) {
                if (hist[bin] >= need || bin == 0) break;
                need -= hist[bin];
            }
            sel_need = need;                       // how many are still wanted inside the chosen bin
            sel_prefix = prefix | (bin << shift);
        }
        __syncthreads();
    }
    const uint32_t kth = sel_prefix;               // key of the k-th largest logit
    const uint32_t need_eq = sel_need;             // how many entries equal to it belong to the top k

    // ---- collect: everything above the threshold, plus the lowest-index `need_eq` ties.
    // Each thread owns a contiguous index range so ties are ranked by index with one block scan.
    const int per = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int i0 = tid * per, i1 = min(V, i0 + per);
    uint32_t eq_local = 0;
    for (int i = i0; i < i1; i++) {
        const uint32_t key = fkey(lr[i]);
        if (key > kth) {
            const uint32_t slot = atomicAdd(&cand_count, 1u);
            if (slot < KMAX) cand[slot] = ((unsigned long long)key << 32) | (uint32_t)(~(uint32_t)i);
        } else if (key == kth) eq_local++;
    }
    scan[tid] = eq_local;
    __syncthreads();
    if (tid == 0) {
        uint32_t run = 0;
        for (int j = 0; j < SAMPLE_THREADS; j++) {
            const uint32_t c = scan[j];
            scan[j] = run;
            run += c;
        }
    }
    __syncthreads();
    uint32_t rank = scan[tid];
    const uint32_t gt_count = cand_count;          // all "greater" entries are in by the barrier above
    __syncthreads();
    for (int i = i0; i < i1 && rank < need_eq; i++) {
        if (fkey(lr[i]) == kth) {
            const uint32_t slot = gt_count + rank;
            if (slot < KMAX) cand[slot] = ((unsigned long long)kth << 32) | (uint32_t)(~(uint32_t)i);
            rank++;
        }
    }
    // the sort works on the next power of two at or above k (at least one entry per thread)
    int nsort = SAMPLE_THREADS;
    while (nsort < (int)k) nsort <<= 1;
    for (int j = tid; j < nsort; j += SAMPLE_THREADS)
        if ((uint32_t)j >= k) cand[j] = 0ull;      // padding sorts last
    __syncthreads();

    // ---- bitonic sort, descending
    for (int size = 2; size <= nsort; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
            for (int j = tid; j < nsort; j += SAMPLE_THREADS) {
                const int partner = j ^ stride;
                if (partner > j) {
                    const bool desc = ((j & size) == 0);
                    const unsigned long long a = cand[j], c = cand[partner];
                    if ((a < c) == desc) cand[j] = c, cand[partner] = a;
                }
            }
            __syncthreads();
        }
    }

    // ---- softmax over the k sorted values / T, then the draw
    const float vmax = fkey_inv((uint32_t)(cand[0] >> 32)) / temperature;
    for (uint32_t j = tid; j < (uint32_t)nsort; j += SAMPLE_THREADS)
        probs[j] = j < k ? expf(fkey_inv((uint32_t)(cand[j] >> 32)) / temperature - vmax) : 0.f;
    __syncthreads();
    float denom = 0.f;
    for (uint32_t j = 0; j < k; j++) denom += probs[j];     // same order on every thread: deterministic
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (uint32_t j = tid; j < k; j += SAMPLE_THREADS) {    // ascending ranks per thread: the first of equal quotients wins
        const float qv = (probs[j] / denom) / noise[(size_t)row * k + j];
        if (qv > bv) bv = qv, bi = (int)j;
    }
    block_argmax(bv, bi, sval, sidx);
    if (tid == 0) {
        const int choice = (bi == 0x7fffffff) ? 0 : bi;
        out_ids[row] = (int64_t)(~(uint32_t)(cand[choice] & 0xffffffffull));
    }
}

// ------------------------------------------------------------------------------------------------
// Any top_k beyond what the candidate sort above holds in LDS (4096 < top_k < V): the whole row is sorted, by a stable
// least-significant-digit radix sort of the indices (three digits of 11 / 11 / 10 bits of the inverted order key, so ascending
// digits are descending logits, and the initial index order makes equal logits come out lowest index first, like
// torch.sort(descending=True, stable=True)).  The two index arrays (uint16: V <= 32768 ... 65536 entries of 2 bytes) and the three
// digit histograms fill the LDS of one CU: 2 * 2 * V + 24 KB.  Counting is done by all four waves in one pass over the row;
// the scatter of a pass must keep the order of equal digits, so one wave walks the sequence 64 entries at a time and ranks the
// lanes of a round among themselves with ballots.  A rarely used path (the reference accepts any k, nanochat/engine.py:147-152):
// correctness over speed, a few hundred microseconds per call.
#define LK_BINS 2048
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_large_k_kernel(const float* __restrict__ logits, int V, int ld, float temperature,
                                                                        int top_k, const float* __restrict__ noise,
                                                                        int64_t* __restrict__ out_ids) {
    extern __shared__ __align__(16) uint8_t lk_lds[];
    __shared__ float sval[4];
    __shared__ int sidx[4];
    __shared__ float fsum[SAMPLE_THREADS];
    uint32_t* hist = (uint32_t*)lk_lds;                                   // [3][LK_BINS]
    uint16_t* ord_a = (uint16_t*)(lk_lds + 3 * LK_BINS * 4);
    uint16_t* ord_b = ord_a + V;
    const int row = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const float* lr = logits + (size_t)row * ld;
    auto digit_of = [](float v, int pass) -> uint32_t {
        const uint32_t inv = ~fkey(v);                                    // ascending inv = descending logit
        return pass == 0 ? (inv & 0x7ffu) : (pass == 1 ? ((inv >> 11) & 0x7ffu) : (inv >> 22));
    };
    // ---- digit counts of all three passes in one scan of the row
    for (int i = tid; i < 3 * LK_BINS; i += SAMPLE_THREADS) hist[i] = 0;
    __syncthreads();
    scan_row(lr, V, tid, [&](float v, int) {
        const uint32_t inv = ~fkey(v);
        atomicAdd(&hist[inv & 0x7ffu], 1u);
        atomicAdd(&hist[LK_BINS + ((inv >> 11) & 0x7ffu)], 1u);
        atomicAdd(&hist[2 * LK_BINS + (inv >> 22)], 1u);
    });
    __syncthreads();
    // ---- exclusive prefix sums, one histogram after the other: thread t owns bins 8t .. 8t+7
    for (int h = 0; h < 3; h++) {
        uint32_t* hh = hist + h * LK_BINS;
        uint32_t local[8], sum = 0;
#pragma unroll
        for (int b = 0; b < 8; b++) local[b] = hh[8 * tid + b], sum += local[b];
        fsum[tid] = __uint_as_float(sum);
        __syncthreads();
        if (tid == 0) {
            uint32_t run = 0;
            for (int t = 0; t < SAMPLE_THREADS; t++) {
                const uint32_t c = __float_as_uint(fsum[t]);
                fsum[t] = __uint_as_float(run);
                run += c;
            }
        }
        __syncthreads();
        uint32_t run = __float_as_uint(fsum[tid]);
#pragma unroll
        for (int b = 0; b < 8; b++) hh[8 * tid + b] = run, run += local[b];
        __syncthreads();
    }
    // ---- three stable scatters by wave 0; indices travel ord_a -> ord_b -> ord_a -> ord_b (the first pass reads the identity)
    if (wave == 0) {
        const unsigned long long lt_mask = lane == 0 ? 0ull : (~0ull >> (64 - lane));
        for (int pass = 0; pass < 3; pass++) {
            const uint16_t* src = (pass & 1) ? ord_b : ord_a;
            uint16_t* dst = (pass & 1) ? ord_a : ord_b;
            volatile uint32_t* offs = hist + pass * LK_BINS;
            for (int base = 0; base < V; base += 4 * 64) {
                // four rounds' worth of indices and logits are asked for at once (the gathers are what a round costs)
                int idx[4];
                float val[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int i = base + 64 * u + lane;
                    idx[u] = i < V ? (pass == 0 ? i : (int)src[i]) : 0;
                }
#pragma unroll
                for (int u = 0; u < 4; u++) val[u] = lr[idx[u]];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const int i = base + 64 * u + lane;
                    const bool valid = i < V;
                    const uint32_t d = digit_of(val[u], pass);
                    unsigned long long peers = __ballot(valid);
#pragma unroll
                    for (int b = 0; b < 11; b++) {
                        const bool bit = (d >> b) & 1u;
                        const unsigned long long bal = __ballot(bit && valid);
                        peers &= bit ? bal : ~bal;
                    }
                    // lanes with the same digit: the lowest of them takes the digit's running offset and moves it on
                    const int rank = __popcll(peers & lt_mask), cnt = __popcll(peers);
                    uint32_t start = 0;
                    if (valid && rank == 0) {
                        start = offs[d];
                        offs[d] = start + (uint32_t)cnt;
                    }
                    const int leader = valid ? (int)__ffsll((long long)peers) - 1 : lane;
                    start = (uint32_t)__shfl((int)start, leader);
                    if (valid) dst[start + rank] = (uint16_t)idx[u];
                    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");      // the next round reads the offsets this one moved
                }
            }
        }
    }
    __syncthreads();
    const uint16_t* order = ord_b;                       // after three passes
    const uint32_t k = (uint32_t)top_k;
    // ---- softmax over the k best / T, then the draw: argmax_j (p_j / denom) / e_j, first j on equal quotients
    const float vmax = lr[order[0]] / temperature;
    float part = 0.f;
    for (uint32_t j = tid; j < k; j += SAMPLE_THREADS) part += expf(lr[order[j]] / temperature - vmax);
    fsum[tid] = part;
    __syncthreads();
    for (int o = SAMPLE_THREADS / 2; o > 0; o >>= 1) {   // a fixed tree: the same sum on every launch
        if (tid < o) fsum[tid] += fsum[tid + o];
        __syncthreads();
    }
    const float denom = fsum[0];
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (uint32_t j = tid; j < k; j += SAMPLE_THREADS) {
        const float qv = (expf(lr[order[j]] / temperature - vmax) / denom) / noise[(size_t)row * k + j];
        if (qv > bv) bv = qv, bi = (int)j;
    }
    block_argmax(bv, bi, sval, sidx);
    if (tid == 0) out_ids[row] = (int64_t)order[(bi == 0x7fffffff) ? 0 : bi];
}

int nc_launch_softcap(const bf16_t* raw, float* out, int64_t n, float softcap, hipStream_t s) {
    NC_CHECK_ARG(raw && out && n >= 0 && softcap > 0.f, "softcap: bad arguments");
    int64_t g = (n + 255) / 256;
    if (g < 1) g = 1;
    if (g > 4096) g = 4096;
    hipLaunchKernelGGL(softcap_kernel, dim3((int)g), dim3(256), 0, s, raw, out, n, softcap);
    NC_CHECK_LAUNCH("softcap");
    return 0;
}

int nc_launch_sample(const float* logits, int B, int V, int ld, float temperature, int top_k, const float* noise,
                     int64_t* out_ids, hipStream_t s) {
    NC_CHECK_ARG(logits && out_ids, "sample: null pointer");
    NC_CHECK_ARG(B > 0 && V > 0 && ld >= V, "sample: bad shape B=%d V=%d ld=%d", B, V, ld);
    NC_CHECK_ARG(temperature >= 0.0f, "sample: temperature must be non-negative");
    NC_CHECK_ARG(temperature == 0.0f || noise, "sample: temperature > 0 needs the exponential noise buffer");
    const int k_eff = (top_k > 0 && top_k < V) ? top_k : 0;
    if (temperature > 0.0f && k_eff > MAX_TOP_K) {
        // the whole row is sorted in the LDS of one CU
        NC_CHECK_ARG(V <= 32768, "sample: top_k %d above %d needs the row's indices in LDS, which holds a vocabulary of at most 32768 (got %d)",
                     top_k, MAX_TOP_K, V);
        const size_t lds_bytes = 3 * LK_BINS * 4 + 2 * (size_t)V * sizeof(uint16_t);
        static bool reserved[64];
        int dev = 0;
        (void)hipGetDevice(&dev);
        if (dev < 0 || dev >= 64 || !reserved[dev]) {
            const hipError_t e = hipFuncSetAttribute((const void*)sample_large_k_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)(3 * LK_BINS * 4 + 4 * 32768));
            if (e != hipSuccess) NC_FAIL(-2, "sample: cannot reserve LDS for the large top_k path: %s", hipGetErrorString(e));
            if (dev >= 0 && dev < 64) reserved[dev] = true;
        }
        NcProfScope prof(4, 4.0 * B * V, s);
        hipLaunchKernelGGL(sample_large_k_kernel, dim3(B), dim3(SAMPLE_THREADS), lds_bytes, s, logits, V, ld, temperature, k_eff, noise, out_ids);
        NC_CHECK_LAUNCH("sample");
        return 0;
    }
    NcProfScope prof(4, 4.0 * B * V, s);
    if (k_eff <= 256)
        hipLaunchKernelGGL(sample_kernel<256>, dim3(B), dim3(SAMPLE_THREADS), 0, s, logits, V, ld, temperature, k_eff, noise, out_ids);
    else
        hipLaunchKernelGGL(sample_kernel<MAX_TOP_K>, dim3(B), dim3(SAMPLE_THREADS), 0, s, logits, V, ld, temperature, k_eff, noise, out_ids);
    NC_CHECK_LAUNCH("sample");
    return 0;
}
