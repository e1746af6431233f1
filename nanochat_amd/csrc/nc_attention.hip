// Split-K attention over the KV cache for newly appended tokens (decode: one token per row).
// Replaces flash_attn_with_kvcache as called at nanochat/gpt.py:113-120 (FA3 signature,
// nanochat/flash_attention.py:139-161): causal, left sliding window of w keys (w+1 keys visible,
// flash_attention.py:91-97), GQA with q head h reading kv head h / (H/Hkv), per-row cache lengths.
// The cache append itself is done by the rotary kernel that runs just before this one.
//
// Layout: q [B*T, H, 128] bf16; k_cache, v_cache [B, Tmax, Hkv, 128] bf16 (one layer).
// A key is 256 contiguous bytes; consecutive keys of one head are Hkv*256 bytes apart.
//
// Mapping: a wave owns a contiguous run of keys of one (row, kv head) or (row, pair of neighbouring kv heads).  16 lanes
// share one key of one head, 16 bytes (8 dims) each, so one 64-lane load instruction fetches four 256-byte segments.  The
// 16-lane dot product is finished with DPP row rotations; each 16-lane group runs its own online softmax
// over the keys it sees (no cross-lane traffic in the loop), and the four groups, then the four waves of
// the workgroup, then the splits (by whichever split-workgroup finishes last, through a counter), are
// merged with the usual (max, sum, acc) rescale.  All G = H/Hkv
// query heads that share the kv head are processed by the same wave so K and V are read exactly once.
//
// HBM traffic per (row, kv head): 2 * n_keys * 256 bytes, the algorithmic minimum.
#include <type_traits>
#include <hip/hip_ext.h>
#include "nc_common.h"
#include "nc_kernels.h"
#include "nc_rope.h"

#define NEG_BIG (-1.0e30f)
#define PART_STRIDE 132     // floats per partial: m, l, pad, pad, acc[128]

// FUSED (decode, one new token per row): the workgroup first finishes its own heads of the q|k|v linear
// (rope_head: partial sums, rotary, QK-norm, value-embedding gate), appends the new key and value to the cache, and
// attends to them out of LDS; the stand-alone rotary/append kernel and the q buffer drop out of the step.  With several
// splits every split finishes the heads for itself (a few KB of partial sums); split 0 alone appends and counts the
// row's own key, the others stream only older keys, so nobody reads the position that is being written.
// HP kv heads per workgroup (1 or 2).  With HP = 2 the two heads are neighbours in memory, a lane group of 32 covers
// both heads of one key (512 contiguous bytes) and a load instruction fetches two keys: the same bytes per instruction in
// runs twice as long, which streams ~8 % faster when there are enough workgroups left.  A lane still serves one head
// (hsel), so the register budget does not change; an odd head count leaves the second half of the last pair idle.
// MODE 0: q is given, the new tokens are already in the cache.  MODE 1: FUSED as described above.  MODE 2: q and the new key and value
// are given finished (flash_attn_with_kvcache(q, k_cache, v_cache, k=, v=), nanochat/flash_attention.py:139-185): the workgroup
// copies its heads of them into LDS, appends key and value to the cache and attends like MODE 1.
template <int G, int MODE, int HP>
__global__ __launch_bounds__(256) void attn_partial_kernel(const bf16_t* __restrict__ q, bf16_t* __restrict__ k_cache,
                                                           bf16_t* __restrict__ v_cache, const int32_t* __restrict__ cache_seqlens,
                                                           int window_left, int seqlens_include_new, bf16_t* __restrict__ out,
                                                           float* __restrict__ partials, uint32_t* __restrict__ counters,
                                                           uint32_t* __restrict__ amax_ws, int T, int H, int Hkv, int Tmax, int nsplit,
                                                           NcRopeSrc rope, int k_min, const float* __restrict__ extra, int n_extra) {
    constexpr bool FUSED = MODE != 0;                    // the row's own token comes from LDS, not from the cache
    constexpr int KPI = 4 / HP;                          // keys per load instruction
    constexpr int TASKS = (G + 2) * HP;                  // FUSED: per head the G query heads, then the new key and value
    __shared__ float merge[4][HP * G][PART_STRIDE];
    __shared__ float fresh[FUSED ? TASKS : 1][128];
    __shared__ int last_flag;
    const int split = blockIdx.x, hp = blockIdx.y, row = blockIdx.z;
    const int b = row / T, t = row % T;
    // the wave index as a scalar: everything derived from it (the head tasks of this wave) then branches instead of predicating
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int grp = lane >> 4, sub = lane & 15;
    const int hsel = grp & (HP - 1), ksel = grp / HP;    // which head of the pair, which key of the instruction
    const int hk = hp * HP + hsel;                       // this lane's kv head
    const bool head_ok = hk < Hkv;
    const int n_heads_here = (hp * HP + HP <= Hkv) ? HP : Hkv - hp * HP;

    // visible keys [lo, hi]
    int pos = cache_seqlens[b];
    if (seqlens_include_new) pos -= T;
    int hi = pos + t;
    if (hi > Tmax - 1) hi = Tmax - 1;
    int lo = (window_left < 0) ? 0 : hi - window_left;
    if (lo < 0) lo = 0;
    // keys below k_min are somebody else's: the shared start of all rows, whose part of the softmax arrives in `extra`
    // (attn_shared_prefix_kernel) and is merged in with the four waves' parts below
    if (lo < k_min) lo = k_min < hi ? k_min : hi;
    // keys streamed from the cache: [lo, k_stop); the fused kernel takes key hi (its own token) from LDS
    const int k_stop = FUSED ? hi : hi + 1;
    const int n_keys = k_stop - lo;
    // contiguous runs, multiples of 4 keys, over nsplit * 4 waves
    const int nw = nsplit * 4;
    int chunk = (n_keys + nw - 1) / nw;
    chunk = (chunk + 3) & ~3;
    const int gw = split * 4 + wave;
    const int k_begin = lo + gw * chunk;
    int k_end = k_begin + chunk;
    if (k_end > k_stop) k_end = k_stop;

    const size_t key_stride = (size_t)Hkv * 128;   // elements between consecutive keys
    const int hk_addr = head_ok ? hk : hp * HP;    // an idle half-pair reads nothing; the address only has to be valid
    const bf16_t* kbase = k_cache + ((size_t)b * Tmax * Hkv + hk_addr) * 128 + sub * 8;
    const bf16_t* vbase = v_cache + ((size_t)b * Tmax * Hkv + hk_addr) * 128 + sub * 8;

    constexpr int UNROLL = 8;     // 8 loads of 1 KB each for K and for V in flight per wave (32 keys of one head, or 16 keys of two)
    uint4 kr[UNROLL], vr[UNROLL];
    // Unconditional loads: a slot past the end of the run re-reads the run's last key (a valid address with finite values) and gets
    // weight zero below, so no lane is masked off and no register is cleared around a load.  The first batch is asked for even by a
    // wave whose run is empty (it reads row 0 and never looks at it): were the fetch behind a branch, the compiler could no longer
    // count the loads in flight and the head tasks below would wait for the keys as well.
    const int k_last = k_end - 1 > 0 ? k_end - 1 : 0;
    auto fetch_k = [&](int kb0) {
#pragma unroll
        for (int i = 0; i < UNROLL; i++) {
            const int j = kb0 + KPI * i + ksel;
            kr[i] = nt_load16(kbase + (size_t)(j < k_end ? j : k_last) * key_stride);
        }
    };
    auto fetch_v = [&](int kb0) {
#pragma unroll
        for (int i = 0; i < UNROLL; i++) {
            const int j = kb0 + KPI * i + ksel;
            vr[i] = nt_load16(vbase + (size_t)(j < k_end ? j : k_last) * key_stride);
        }
    };
    // Loads return in issue order, so the few KB that the head tasks of this wave need go out first and the first batch of keys
    // right behind them: the rotary/norm arithmetic then runs while the keys are still on their way.
    // Wave w finishes head task w, w+4, ...: per head of the pair, tasks 0..G-1 are the query heads, G the key head, G+1 the
    // value head.
    constexpr int TASKS_PER_WAVE = (TASKS + 3) / 4;
    RopeRaw<4> raw[MODE == 1 ? TASKS_PER_WAVE : 1];
    uint32_t plain1[MODE == 2 ? TASKS_PER_WAVE : 1], plain2[MODE == 2 ? TASKS_PER_WAVE : 1];
    auto task_head = [&](int task) {
        const int th = task / (G + 2), tt = task % (G + 2), thk = hp * HP + th;
        return tt < G ? thk * G + tt : (tt == G ? H + thk : H + Hkv + thk);
    };
    AmaxWords amax_words = {};
    if (MODE == 1) {
        if (rope.pq.parts) amax_words = amax_load_scalar(rope.pq.a_amax);
#pragma unroll
        for (int i = 0; i < TASKS_PER_WAVE; i++) {
            const int task = wave + 4 * i;
            if (task < (G + 2) * n_heads_here) rope_head_load(rope, row, hi, task_head(task), H, Hkv, lane, raw[i]);
        }
    }
    if (MODE == 2) {
#pragma unroll
        for (int i = 0; i < TASKS_PER_WAVE; i++) {
            const int task = wave + 4 * i;
            plain1[i] = plain2[i] = 0u;
            if (task < (G + 2) * n_heads_here) {
                const int tt = task % (G + 2), thk = hp * HP + task / (G + 2);
                const bf16_t* src = tt < G ? q + ((size_t)row * H + thk * G + tt) * 128
                                           : (tt == G ? rope.k_new : rope.v_new) + ((size_t)row * Hkv + thk) * 128;
                plain1[i] = src[lane], plain2[i] = src[lane + 64];
            }
        }
    }
    fetch_k(k_begin < k_end ? k_begin : 0);
    fetch_v(k_begin < k_end ? k_begin : 0);

    if (FUSED) {
        const float a_amax = amax_from_words(amax_words);
#pragma unroll
        for (int i = 0; i < TASKS_PER_WAVE; i++) {
            const int task = wave + 4 * i;
            if (task < (G + 2) * n_heads_here) {
                const int tt = task % (G + 2), thk = hp * HP + task / (G + 2);
                float y1, y2;
                if (MODE == 1) rope_head_finish(rope, row, task_head(task), H, Hkv, lane, raw[i], a_amax, y1, y2);
                else y1 = bf16_to_f32((bf16_t)plain1[i]), y2 = bf16_to_f32((bf16_t)plain2[i]);
                fresh[task][lane] = y1, fresh[task][lane + 64] = y2;
                if (tt >= G && split == 0 && hi >= 0 && hi < Tmax) {
                    bf16_t* dst = (tt == G ? k_cache : v_cache) + (((size_t)b * Tmax + hi) * Hkv + thk) * 128;
                    dst[lane] = f32_to_bf16(y1);
                    dst[lane + 64] = f32_to_bf16(y2);
                }
            }
        }
        __syncthreads();
    }
    const int fbase = (head_ok ? hsel : 0) * (G + 2);     // this lane's head inside fresh[]

    // q for the G heads of this kv head, pre-scaled by log2(e) / sqrt(128)
    const float qscale = 1.4426950408889634f * 0.08838834764831845f;
    float qf[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        if (FUSED) {
#pragma unroll
            for (int e = 0; e < 8; e++) qf[g][e] = fresh[fbase + g][sub * 8 + e] * qscale;
        } else {
            const uint4 qv = *(const uint4*)(q + ((size_t)row * H + hk_addr * G + g) * 128 + sub * 8);
            const uint32_t w[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
            for (int j = 0; j < 4; j++) {
                qf[g][2 * j] = bf16_lo(w[j]) * qscale;
                qf[g][2 * j + 1] = bf16_hi(w[j]) * qscale;
            }
        }
    }
    float m[G], l[G], acc[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
        m[g] = NEG_BIG, l[g] = 0.f;
#pragma unroll
        for (int d = 0; d < 8; d++) acc[g][d] = 0.f;
    }
    if (FUSED) {
        // the row's own key: the lanes of wave 0 that hold key slot 0 start their running softmax from it (weight exp2(0) = 1)
#pragma unroll
        for (int g = 0; g < G; g++) {
            float d = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) d = fmaf(qf[g][e], fresh[fbase + G][sub * 8 + e], d);
            d = row16_sum(d);
            if (split == 0 && wave == 0 && ksel == 0 && head_ok) {
                m[g] = d, l[g] = 1.f;
#pragma unroll
                for (int e = 0; e < 8; e++) acc[g][e] = fresh[fbase + G + 1][sub * 8 + e];
            }
        }
    }

    // One batch of keys: scores from kr, then (all but the last batch) the next batch's keys are asked for while the softmax and
    // the value sums of this one run, and the next values once vr is free.  The last batch is a copy of the body without the
    // prefetch, not a branch inside it: behind a branch the compiler could not count the loads in flight.
    auto batch = [&](int kb0, auto prefetch) {
        bool ok[UNROLL];
        float sc[G][UNROLL];
#pragma unroll
        for (int i = 0; i < UNROLL; i++) {
            ok[i] = kb0 + KPI * i + ksel < k_end && head_ok;
            const uint32_t w[4] = {kr[i].x, kr[i].y, kr[i].z, kr[i].w};
            float kf[8];
#pragma unroll
            for (int j = 0; j < 4; j++) kf[2 * j] = bf16_lo(w[j]), kf[2 * j + 1] = bf16_hi(w[j]);
#pragma unroll
            for (int g = 0; g < G; g++) {
                float d = 0.f;
#pragma unroll
                for (int e = 0; e < 8; e++) d = fmaf(qf[g][e], kf[e], d);
                d = row16_sum(d);
                sc[g][i] = ok[i] ? d : NEG_BIG;
            }
        }
        if (decltype(prefetch)::value) fetch_k(kb0 + KPI * UNROLL);
#pragma unroll
        for (int g = 0; g < G; g++) {
            float mn = m[g];
#pragma unroll
            for (int i = 0; i < UNROLL; i++) mn = fmaxf(mn, sc[g][i]);
            const float corr = exp2f(m[g] - mn);
            m[g] = mn;
            l[g] *= corr;
#pragma unroll
            for (int d = 0; d < 8; d++) acc[g][d] *= corr;
#pragma unroll
            for (int i = 0; i < UNROLL; i++) sc[g][i] = ok[i] ? exp2f(sc[g][i] - mn) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < UNROLL; i++) {
            const uint32_t w[4] = {vr[i].x, vr[i].y, vr[i].z, vr[i].w};
            float vf[8];
#pragma unroll
            for (int j = 0; j < 4; j++) vf[2 * j] = bf16_lo(w[j]), vf[2 * j + 1] = bf16_hi(w[j]);
#pragma unroll
            for (int g = 0; g < G; g++) {
                l[g] += sc[g][i];
#pragma unroll
                for (int d = 0; d < 8; d++) acc[g][d] = fmaf(sc[g][i], vf[d], acc[g][d]);
            }
        }
        if (decltype(prefetch)::value) fetch_v(kb0 + KPI * UNROLL);
    };
    if (k_begin < k_end) {
        int kb0 = k_begin;
        for (; kb0 + KPI * UNROLL < k_end; kb0 += KPI * UNROLL) batch(kb0, std::true_type{});
        batch(kb0, std::false_type{});
    }

    // merge the 16-lane groups of the wave that serve the same head (all four, or the two with the same hsel)
#pragma unroll
    for (int g = 0; g < G; g++) {
        float mm = m[g];
        if (HP == 1) mm = fmaxf(mm, __shfl_xor(mm, 16));
        mm = fmaxf(mm, __shfl_xor(mm, 32));
        const float w = exp2f(m[g] - mm);
        float lw = l[g] * w;
        if (HP == 1) lw += __shfl_xor(lw, 16);
        lw += __shfl_xor(lw, 32);
#pragma unroll
        for (int d = 0; d < 8; d++) {
            float a = acc[g][d] * w;
            if (HP == 1) a += __shfl_xor(a, 16);
            a += __shfl_xor(a, 32);
            acc[g][d] = a;
        }
        m[g] = mm, l[g] = lw;
        if (ksel == 0) {
            if (sub == 0) merge[wave][hsel * G + g][0] = mm, merge[wave][hsel * G + g][1] = lw;
#pragma unroll
            for (int d = 0; d < 8; d++) merge[wave][hsel * G + g][4 + sub * 8 + d] = acc[g][d];
        }
    }
    __syncthreads();

    // merge the four waves: thread (head of the pair, g, d) for d < 128
    float am = 0.f;
    for (int item = threadIdx.x; item < n_heads_here * G * 128; item += 256) {
        const int hg = item >> 7, d = item & 127;           // hg = (head of the pair) * G + g
        float mm = NEG_BIG;
#pragma unroll
        for (int w = 0; w < 4; w++) mm = fmaxf(mm, merge[w][hg][0]);
        const int head = (hp * HP + hg / G) * G + hg % G;
        const float* ex = extra ? extra + ((size_t)row * H + head) * n_extra * PART_STRIDE : nullptr;
        // up to 16 partial results of the shared start: all of their words asked for at once (one trip to memory at the end of the
        // kernel instead of one per partial), added in chunk order like the loop below
        const bool few = ex && n_extra <= 16;
        float em[16], el[16], ea[16];
        if (few) {
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const float* q = ex + (e < n_extra ? e : 0) * PART_STRIDE;
                em[e] = q[0], el[e] = q[1], ea[e] = q[4 + d];
            }
#pragma unroll
            for (int e = 0; e < 16; e++)
                if (e < n_extra) mm = fmaxf(mm, em[e]);
        } else if (ex) {
            for (int e = 0; e < n_extra; e++) mm = fmaxf(mm, ex[e * PART_STRIDE]);
        }
        float ls = 0.f, a = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float sc = exp2f(merge[w][hg][0] - mm);
            ls += merge[w][hg][1] * sc;
            a += merge[w][hg][4 + d] * sc;
        }
        if (few) {
#pragma unroll
            for (int e = 0; e < 16; e++)
                if (e < n_extra) {
                    const float sc = exp2f(em[e] - mm);
                    ls += el[e] * sc;
                    a += ea[e] * sc;
                }
        } else if (ex) {
            for (int e = 0; e < n_extra; e++) {
                const float sc = exp2f(ex[e * PART_STRIDE] - mm);
                ls += ex[e * PART_STRIDE + 1] * sc;
                a += ex[e * PART_STRIDE + 4 + d] * sc;
            }
        }
        if (nsplit == 1) {
            const bf16_t o = f32_to_bf16(a / ls);
            out[((size_t)row * H + head) * 128 + d] = o;
            am = amax_fold(am, bf16_to_f32(o));
        } else {
            float* p = partials + (((size_t)row * H + head) * nsplit + split) * PART_STRIDE;
            if (d == 0) coherent_store_f1(p, mm), coherent_store_f1(p + 1, ls);
            coherent_store_f1(p + 4 + d, a);
        }
    }
    if (nsplit > 1) {
        // the split that arrives last at this (row, head pair) merges all of them, in split order
        if (!arrive_and_check_last(&counters[row * Hkv + hp * HP], (uint32_t)nsplit, &last_flag)) return;
        for (int item = threadIdx.x; item < n_heads_here * G * 128; item += 256) {
            const int hg = item >> 7, d = item & 127;
            const int head = (hp * HP + hg / G) * G + hg % G;
            const float* p = partials + ((size_t)row * H + head) * nsplit * PART_STRIDE;
            float mm = NEG_BIG;
            for (int sidx = 0; sidx < nsplit; sidx++) mm = fmaxf(mm, coherent_load_f1(p + sidx * PART_STRIDE));
            float ls = 0.f, a = 0.f;
            for (int sidx = 0; sidx < nsplit; sidx++) {
                const float sc = exp2f(coherent_load_f1(p + sidx * PART_STRIDE) - mm);
                ls += coherent_load_f1(p + sidx * PART_STRIDE + 1) * sc;
                a += coherent_load_f1(p + sidx * PART_STRIDE + 4 + d) * sc;
            }
            const bf16_t o = f32_to_bf16(a / ls);
            out[((size_t)row * H + head) * 128 + d] = o;
            am = amax_fold(am, bf16_to_f32(o));
        }
        if (threadIdx.x == 0) __hip_atomic_store(&counters[row * Hkv + hp * HP], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (amax_ws) {
        // one publication per workgroup (only the first threads hold output values)
        am = wave_amax(am);
        __syncthreads();
        if (lane == 0) merge[wave][0][0] = am;
        __syncthreads();
        if (threadIdx.x == 0) amax_publish(amax_ws, amax_join(amax_join(merge[0][0][0], merge[1][0][0]), amax_join(merge[2][0][0], merge[3][0][0])));
    }
}

// ------------------------------------------------------------------------------------------------
// Two kv heads per workgroup when the head pairs alone still give the chip ~6 waves per CU (512-byte runs stream faster
// than 256-byte ones only if enough workgroups remain).
static int pick_heads_per_wg(int B, int T, int Hkv) { return (Hkv >= 2 && (long)B * T * ((Hkv + 1) / 2) * 4 >= 1536) ? 2 : 1; }

static int pick_splits(int B, int T, int Hkv, int max_keys) {
    // One split whenever the (row, kv head or head pair) workgroups alone give every CU ~6-8 waves: measured at batch 64 x 13 heads,
    // one split streams 513 keys at 5.9 TB/s and 2048 keys at 5.6 TB/s, and every extra split only adds merge work.
    // Small batches need the splits to fill the machine; keep at least 64 keys per wave.
    const int hp = pick_heads_per_wg(B, T, Hkv);
    if (hp == 2) return 1;
    const long base_waves = (long)B * T * Hkv * 4;
    int s = 1;
    while (s < 16 && base_waves * s < 2048 && max_keys / (4 * s * 2) >= 64) s *= 2;
    return s;
}

// arrival counters, one per (row, kv head), zero between launches; split partials for up to 16 splits
size_t nc_attn_counter_bytes(int B, int T, int H) { return (((size_t)B * T * H * sizeof(uint32_t)) + 255) & ~(size_t)255; }
size_t nc_attn_partial_bytes(int B, int T, int H) { return (size_t)B * T * H * 16 * PART_STRIDE * sizeof(float); }

int nc_attn_splits(int B, int T, int Hkv, int window_left, int Tmax) {
    const int max_keys = (window_left >= 0 && window_left + 1 < Tmax) ? window_left + 1 : Tmax;
    return pick_splits(B, T, Hkv, max_keys);
}

// mode 0: q given, new tokens already in the cache.  mode 1: *rope names the raw q|k|v rows (rotary, QK-norm, value embedding and the
// append are done here).  mode 2: q given, rope->k_new / rope->v_new hold the finished new key and value, appended here.
static int launch_attention_impl(const bf16_t* q, const NcRopeSrc* rope, int mode, bf16_t* k_cache, bf16_t* v_cache,
                                 const int32_t* cache_seqlens, int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax,
                                 int seqlens_include_new, uint32_t* counters, void* partials, size_t partial_bytes, uint32_t* amax_ws,
                                 int force_splits, int counters_are_zero, hipStream_t s, int k_min = 0, const float* extra = nullptr,
                                 int n_extra = 0) {
    NC_CHECK_ARG((q || mode == 1) && k_cache && v_cache && cache_seqlens && out, "decode_attention: null pointer");
    // many queries per row: the matrix-core kernel (a workgroup there covers 128 queries; below 16 queries per row
    // the per-query streaming kernel wastes less)
    if (mode == 0 && T >= 16 && force_splits <= 0)
        return nc_launch_attention_prefill(q, k_cache, v_cache, cache_seqlens, window_left, out, B, T, H, Hkv, Tmax, seqlens_include_new,
                                           amax_ws, s);
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0 && Hkv > 0 && Tmax > 0, "decode_attention: bad shape");
    NC_CHECK_ARG(H % Hkv == 0, "decode_attention: n_head %d not a multiple of n_kv_head %d", H, Hkv);
    const int G = H / Hkv;
    NC_CHECK_ARG(G == 1 || G == 2 || G == 4 || G == 8, "decode_attention: query group size %d not in {1,2,4,8}", G);
    NC_CHECK_ARG((long)B * T <= 65535 && Hkv <= 65535, "decode_attention: more than 65535 query rows in one launch");
    NC_CHECK_ARG((!q || ((uintptr_t)q & 15) == 0) && ((uintptr_t)k_cache & 15) == 0 && ((uintptr_t)v_cache & 15) == 0,
                 "decode_attention: pointers must be 16-byte aligned");
    int max_keys = (window_left >= 0 && window_left + 1 < Tmax) ? window_left + 1 : Tmax;
    int nsplit = force_splits > 0 ? force_splits : pick_splits(B, T, Hkv, max_keys);
    NC_CHECK_ARG(nsplit >= 1 && nsplit <= 16, "decode_attention: splits must be 1..16");
    if (mode != 0) {
        NC_CHECK_ARG(rope && T == 1 && !seqlens_include_new, "decode_attention: the in-kernel append needs one new token per row, not yet counted");
    }
    if (mode == 1) {
        NC_CHECK_ARG((rope->qkv || rope->pq.parts) && rope->cos_t && rope->sin_t && rope->rope_len > 0, "decode_attention: rotary source missing");
        NC_CHECK_ARG(!rope->ve_table || (rope->ve_gate_w && rope->xn && rope->idx && rope->ld_xn >= 12),
                     "decode_attention: value embedding needs gate weights, xn and idx");
    }
    if (mode == 2) NC_CHECK_ARG(rope->k_new && rope->v_new, "decode_attention: new key / value missing");
    if (nsplit > 1) {
        const size_t need = (size_t)B * T * H * nsplit * PART_STRIDE * sizeof(float);
        NC_CHECK_ARG(counters && partials && partial_bytes >= need, "decode_attention: %zu bytes of split workspace needed, %zu given",
                     need, partial_bytes);
        NC_CHECK_ARG(((uintptr_t)partials & 15) == 0, "decode_attention: workspace must be 16-byte aligned");
        if (!counters_are_zero) nc_clear_u32(counters, B * T * Hkv, s);
    }
    NC_CHECK_ARG(!extra || (nsplit == 1 && mode == 0 && T == 1 && n_extra > 0 && k_min > 0),
                 "decode_attention: a shared first part goes with one split, one query per row and tokens already appended");
    // when the profiler is on, the launch carries its own event pair (kernel begin / end, no marker packets around it)
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    const bool timed = nc_prof_take(0, 0.0, 0, &ev0, &ev1);
    float* parts = (float*)partials;
    const int hp = (force_splits > 0 || nsplit > 1) ? 1 : pick_heads_per_wg(B, T, Hkv);
    dim3 grid(nsplit, hp == 2 ? (Hkv + 1) / 2 : Hkv, B * T), block(256);
    const NcRopeSrc none{};
    const NcRopeSrc& rs = rope ? *rope : none;
#define LAUNCH_GMH(GG, MM, HH)                                                                                                     \
    do {                                                                                                                           \
        if (timed)                                                                                                                 \
            hipExtLaunchKernelGGL((attn_partial_kernel<GG, MM, HH>), grid, block, 0, s, ev0, ev1, 0, q, k_cache, v_cache,         \
                                  cache_seqlens, window_left, seqlens_include_new, out, parts, counters, amax_ws, T, H, Hkv, Tmax, \
                                  nsplit, rs, k_min, extra, n_extra);                                                              \
        else                                                                                                                       \
            hipLaunchKernelGGL((attn_partial_kernel<GG, MM, HH>), grid, block, 0, s, q, k_cache, v_cache, cache_seqlens,           \
                               window_left, seqlens_include_new, out, parts, counters, amax_ws, T, H, Hkv, Tmax, nsplit, rs,       \
                               k_min, extra, n_extra);                                                                             \
    } while (0)
#define LAUNCH_GH(GG, HH)                          \
    do {                                           \
        if (mode == 1) LAUNCH_GMH(GG, 1, HH);      \
        else if (mode == 2) LAUNCH_GMH(GG, 2, HH); \
        else LAUNCH_GMH(GG, 0, HH);                \
    } while (0)
#define LAUNCH_G(GG)                   \
    do {                               \
        if (hp == 2) LAUNCH_GH(GG, 2); \
        else LAUNCH_GH(GG, 1);         \
    } while (0)
    if (G == 1) LAUNCH_G(1);
    else if (G == 2) LAUNCH_G(2);
    else if (G == 4) LAUNCH_G(4);
    else LAUNCH_G(8);
#undef LAUNCH_G
#undef LAUNCH_GH
#undef LAUNCH_GMH
    NC_CHECK_LAUNCH("decode_attention");
    return 0;
}

// What a launch with these shapes does: the number of key splits and the kv heads per workgroup (1 or 2).  `in_kernel_append`:
// the decode forms that finish / append the new token themselves (they never take the many-queries kernel).
void nc_attention_plan(int B, int T, int Hkv, int window_left, int Tmax, int force_splits, int* splits_out, int* heads_per_wg_out) {
    const int max_keys = (window_left >= 0 && window_left + 1 < Tmax) ? window_left + 1 : Tmax;
    const int nsplit = force_splits > 0 ? force_splits : pick_splits(B, T, Hkv, max_keys);
    if (splits_out) *splits_out = nsplit;
    if (heads_per_wg_out) *heads_per_wg_out = (force_splits > 0 || nsplit > 1) ? 1 : pick_heads_per_wg(B, T, Hkv);
}

int nc_launch_attention(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens,
                        int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                        uint32_t* counters, void* partials, size_t partial_bytes, uint32_t* amax_ws, int force_splits,
                        int counters_are_zero, hipStream_t s) {
    return launch_attention_impl(q, nullptr, 0, const_cast<bf16_t*>(k_cache), const_cast<bf16_t*>(v_cache), cache_seqlens, window_left, out,
                                 B, T, H, Hkv, Tmax, seqlens_include_new, counters, partials, partial_bytes, amax_ws, force_splits,
                                 counters_are_zero, s);
}

// Decode step, one new token per row, cache_seqlens not yet counting it: finish the q|k|v linear (rotary, QK-norm,
// value embedding), append key and value at cache_seqlens[b], attend.  counters / partials as for nc_launch_attention.
int nc_launch_attention_fused(NcRopeSrc rope, bf16_t* k_cache, bf16_t* v_cache, const int32_t* cache_seqlens, int window_left,
                              bf16_t* out, int B, int H, int Hkv, int Tmax, uint32_t* counters, void* partials, size_t partial_bytes,
                              uint32_t* amax_ws, int force_splits, int counters_are_zero, hipStream_t s) {
    return launch_attention_impl(nullptr, &rope, 1, k_cache, v_cache, cache_seqlens, window_left, out, B, 1, H, Hkv, Tmax, 0, counters,
                                 partials, partial_bytes, amax_ws, force_splits, counters_are_zero, s);
}

// Decode attention for rows that share their first `shared_len` cached tokens (one prompt replicated to every row,
// nanochat/engine.py:198-214) and sit at the same position: the shared keys are read once for all rows on the matrix cores
// (attn_shared_prefix_kernel, from row 0 of the cache), the per-row kernel streams only each row's own tail [shared_len, p] and merges
// the two parts.  One new token per row, already appended.  shared_parts: nc_attn_shared_partial_bytes() bytes.  The per-row launch
// takes one workgroup per (row, kv head) whatever the batch: a row's own tail is short, and the merge of the shared part belongs to the
// workgroup that has the row.
int nc_launch_attention_shared(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int shared_len,
                               int window_left, bf16_t* out, int B, int H, int Hkv, int Tmax, int seqlens_include_new, void* shared_parts,
                               size_t shared_part_bytes, uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(B > 0 && H > 0 && Hkv > 0 && Tmax > 0 && H % Hkv == 0, "decode_attention_shared: bad shape");
    NC_CHECK_ARG(shared_len > 0 && shared_len < Tmax, "decode_attention_shared: shared length %d outside (0, %d)", shared_len, Tmax);
    int nchunks = 0;
    int rc = nc_launch_attention_shared_prefix(q, k_cache, v_cache, cache_seqlens, shared_len, window_left, seqlens_include_new,
                                               (float*)shared_parts, shared_part_bytes, B, H, Hkv, Tmax, &nchunks, s);
    if (rc) return rc;
    // (one split whatever the batch: a row's own tail is short, and the merge of the shared part belongs to the workgroup that has the row)
    return launch_attention_impl(q, nullptr, 0, const_cast<bf16_t*>(k_cache), const_cast<bf16_t*>(v_cache), cache_seqlens, window_left, out, B, 1,
                                 H, Hkv, Tmax, seqlens_include_new, nullptr, nullptr, 0, amax_ws, 1, 1, s, shared_len, (const float*)shared_parts,
                                 nchunks);
}

// cache[b, cache_seqlens[b] + t] = new[b, t] for keys and values (nanochat/flash_attention.py:167-170 with per-row positions);
// positions outside [0, Tmax) are skipped.  token_elems = Hkv * 128.
__global__ void kv_append_kernel(const bf16_t* __restrict__ k_new, const bf16_t* __restrict__ v_new, bf16_t* __restrict__ k_cache,
                                 bf16_t* __restrict__ v_cache, const int32_t* __restrict__ cache_seqlens, int T, int Tmax, int token_elems) {
    const int b = blockIdx.y, t = blockIdx.x;
    const int pos = cache_seqlens[b] + t;
    if (pos < 0 || pos >= Tmax) return;
    const uint4* ks = (const uint4*)(k_new + ((size_t)b * T + t) * token_elems);
    const uint4* vs = (const uint4*)(v_new + ((size_t)b * T + t) * token_elems);
    uint4* kd = (uint4*)(k_cache + ((size_t)b * Tmax + pos) * token_elems);
    uint4* vd = (uint4*)(v_cache + ((size_t)b * Tmax + pos) * token_elems);
    for (int i = threadIdx.x; i < token_elems / 8; i += blockDim.x) kd[i] = ks[i], vd[i] = vs[i];
}

// flash_attn_with_kvcache(q, k_cache, v_cache, k=k_new, v=v_new, cache_seqlens=...): append, then attend.  One new token per row
// is appended by the attention workgroups themselves; several go through a copy kernel and the ordinary kernels.
int nc_launch_attention_append(const bf16_t* q, const bf16_t* k_new, const bf16_t* v_new, bf16_t* k_cache, bf16_t* v_cache,
                               const int32_t* cache_seqlens, int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax,
                               uint32_t* counters, void* partials, size_t partial_bytes, uint32_t* amax_ws, int force_splits,
                               hipStream_t s) {
    NC_CHECK_ARG(q && k_new && v_new && k_cache && v_cache && cache_seqlens && out, "attention_append: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0 && Hkv > 0 && Tmax > 0 && B <= 65535, "attention_append: bad shape");
    NC_CHECK_ARG((((uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0,
                 "attention_append: pointers must be 16-byte aligned");
    if (T == 1) {
        NcRopeSrc src{};
        src.k_new = k_new, src.v_new = v_new;
        return launch_attention_impl(q, &src, 2, k_cache, v_cache, cache_seqlens, window_left, out, B, 1, H, Hkv, Tmax, 0, counters, partials,
                                     partial_bytes, amax_ws, force_splits, 0, s);
    }
    hipLaunchKernelGGL(kv_append_kernel, dim3(T, B), dim3(Hkv * 16 < 256 ? Hkv * 16 : 256), 0, s, k_new, v_new, k_cache, v_cache,
                       cache_seqlens, T, Tmax, Hkv * 128);
    NC_CHECK_LAUNCH("kv_append");
    return launch_attention_impl(q, nullptr, 0, k_cache, v_cache, cache_seqlens, window_left, out, B, T, H, Hkv, Tmax, 0, counters, partials,
                                 partial_bytes, amax_ws, force_splits, 0, s);
}

// ------------------------------------------------------------------------------------------------
// The same attention for callers that cannot allocate and have no workspace to bring (code under HIP graph capture, tight serving
// loops): the split counters and partial results live in a file-scope device array instead of a caller's buffer.  Every GPU the
// library runs on holds its own copy of the array, at its own address, until the process ends; the address is looked up once per
// device, with that device current, and only that looked-up pointer is ever handed to a kernel (the array's name in host code is
// a host-side stand-in, not a device address).  All calls on one GPU share the array: calls that overlap there race.
#define NC_STATIC_ATTN_MAX_ROW_HEADS 1024     // B * T * H at most: 1024 * (16 splits * 132 floats + one counter)
#define NC_STATIC_ATTN_COUNTER_BYTES ((size_t)NC_STATIC_ATTN_MAX_ROW_HEADS * sizeof(uint32_t))
#define NC_STATIC_ATTN_PARTIAL_BYTES ((size_t)NC_STATIC_ATTN_MAX_ROW_HEADS * 16 * PART_STRIDE * sizeof(float))
static __device__ __align__(256) unsigned char scratch[NC_STATIC_ATTN_COUNTER_BYTES + NC_STATIC_ATTN_PARTIAL_BYTES];

#define NC_MAX_DEVICES 64
static void* g_scratch_ptr[NC_MAX_DEVICES];      // per device: the address of that device's copy of scratch[]

// The device-side address of scratch[] on the current device, or nullptr after nc_set_error().
static void* static_scratch_for_current_device() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= NC_MAX_DEVICES) {
        nc_set_error("decode_attention_static: no current device (or more than %d devices)", NC_MAX_DEVICES);
        return nullptr;
    }
    void* p = __atomic_load_n(&g_scratch_ptr[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            nc_set_error("decode_attention_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        __atomic_store_n(&g_scratch_ptr[dev], p, __ATOMIC_RELEASE);    // two threads racing here look up the same address
    }
    return p;
}

size_t nc_attention_static_max_row_heads(void) { return NC_STATIC_ATTN_MAX_ROW_HEADS; }

int nc_launch_attention_static(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int window_left,
                               bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new, uint32_t* amax_ws,
                               int force_splits, hipStream_t s) {
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0, "decode_attention_static: bad shape");
    NC_CHECK_ARG((long)B * T * H <= NC_STATIC_ATTN_MAX_ROW_HEADS,
                 "decode_attention_static: %ld (row, head) pairs exceed the built-in scratch of %d; use nc_decode_attention with a workspace",
                 (long)B * T * H, NC_STATIC_ATTN_MAX_ROW_HEADS);
    unsigned char* base = (unsigned char*)static_scratch_for_current_device();
    if (!base) return -2;
    // the counters are cleared by a small fill kernel inside the launch (what the previous call left there is not trusted)
    return launch_attention_impl(q, nullptr, 0, const_cast<bf16_t*>(k_cache), const_cast<bf16_t*>(v_cache), cache_seqlens, window_left, out, B,
                                 T, H, Hkv, Tmax, seqlens_include_new, (uint32_t*)base, base + NC_STATIC_ATTN_COUNTER_BYTES,
                                 NC_STATIC_ATTN_PARTIAL_BYTES, amax_ws, force_splits, 0, s);
}
