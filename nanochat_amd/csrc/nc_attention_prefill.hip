// Attention of many query positions per row over the KV cache (prefill): the T > 1 case of
// flash_attn_with_kvcache (nanochat/flash_attention.py:139-185) and of flash_attn_func (:115-136), causal with an
// optional left window, GQA by kv head = q head / (H / Hkv), head_dim 128, bf16 in, fp32 softmax, bf16 out.
// The new keys and values are already in the cache (qkv_rope_append); a query at cache position p sees keys
// [max(0, p - window), p].
//
// Flash-attention forward on the bf16 matrix cores, written "transposed" so that nothing has to move between lanes:
//   S^T = K . Q^T   (v_mfma_f32_32x32x16_bf16, A = K rows from LDS, B = the wave's 32 queries held in registers):
//                   a lane ends up with 16 scores of ONE query (column lane % 32), so the running max / sum of the
//                   online softmax are per-lane scalars plus one exchange with lane ^ 32;
//   O^T = V^T . P^T (same instruction, A = V^T from LDS, B = P^T): the B operand is exactly the S^T accumulator
//                   registers converted to bf16 (the key order inside a 16-key chunk is the accumulator's row order,
//                   and V^T is read in that order), and the output columns are again the lane's own query, so the
//                   softmax rescale is a per-lane multiply.
// A workgroup is 4 waves x 32 queries of one (row, head); keys go through LDS in blocks of 32: K as [key][d]
// (rows padded to 272 B), V transposed to [d][key] (rows padded to 72 B) while it is staged.  The loads of the next
// block are in flight while the current one is multiplied.
#include "nc_common.h"
#include "nc_kernels.h"

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

#define PF_KPITCH 272          // bytes per K row in LDS (256 + 16)
#define PF_VPITCH 72           // bytes per V^T row in LDS (64 + 8)
#define PF_NEG (-1.0e30f)

__device__ __forceinline__ v8bf as_v8bf(uint4 v) { return __builtin_bit_cast(v8bf, v); }

// GS = query heads of one kv head that share a workgroup (1, 2 or 4): wave w serves head (w % GS) of the group and the (w / GS)-th
// block of 32 queries, so a workgroup covers 128 / GS queries of GS heads and the keys and values it stages are used by all of them.
// Keys go through LDS 64 at a time (two sub-blocks of 32, each laid out and multiplied as described above): one pair of barriers and
// one round of loads in flight per 64 keys.  A wave skips a sub-block that none of its queries can see (past the causal diagonal, or
// wholly before the window of its first query).  Tiles are handed out from the end of the sequence, longest key ranges first.
template <int GS>
__global__ __launch_bounds__(256) void attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache,
                                                           const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ cache_seqlens,
                                                           int window_left, int seqlens_include_new, bf16_t* __restrict__ out,
                                                           uint32_t* __restrict__ amax_ws, int T, int H, int Hkv, int Tmax) {
    constexpr int QT = 128 / GS;                               // queries per workgroup
    __shared__ __align__(16) uint8_t lds_k[2][32 * PF_KPITCH];
    __shared__ __align__(16) uint8_t lds_v[2][128 * PF_VPITCH];
    __shared__ float red[4];
    const int G = H / Hkv, parts = G / GS;                     // workgroups per kv head along the head axis
    const int qb0 = ((int)gridDim.x - 1 - (int)blockIdx.x) * QT, hk = blockIdx.y / parts, b = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int h = hk * G + (blockIdx.y % parts) * GS + wave % GS;
    const int qw0 = qb0 + (wave / GS) * 32;                    // first query of this wave
    const int col = lane & 31, hl = lane >> 5;

    int pos0 = cache_seqlens[b];
    if (seqlens_include_new) pos0 -= T;
    // this lane's query
    const int t = qw0 + col;
    const bool q_ok = t < T;
    const int qpos = pos0 + (q_ok ? t : T - 1);
    const int q_lo = window_left < 0 ? 0 : max(0, qpos - window_left);
    // what the wave as a whole can see: keys [w_lo, w_hi]
    const int w_hi = pos0 + min(qw0 + 31, T - 1);
    const int w_lo = window_left < 0 ? 0 : max(0, pos0 + min(qw0, T - 1) - window_left);

    // key range of the workgroup
    const int t_last = min(qb0 + QT - 1, T - 1);
    int k_hi = pos0 + t_last;
    if (k_hi > Tmax - 1) k_hi = Tmax - 1;
    int k_lo = window_left < 0 ? 0 : pos0 + qb0 - window_left;
    if (k_lo < 0) k_lo = 0;
    const int kb_first = k_lo & ~63;

    // Q fragments: B operand of K.Q^T, lane = (query col, d half hl): Q[query][16c + 8hl .. +7]
    v8bf qf[8];
    {
        const bf16_t* qrow = q + (((size_t)b * T + (q_ok ? t : T - 1)) * H + h) * 128;
#pragma unroll
        for (int c = 0; c < 8; c++) qf[c] = as_v8bf(*(const uint4*)(qrow + 16 * c + 8 * hl));
    }

    v16f o[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] = 0.f;
    float m_run = PF_NEG, l_run = 0.f;
    const float sc = 1.4426950408889634f * 0.08838834764831845f;     // log2(e) / sqrt(128)

    // staging: thread = (16-byte chunk ch of a key, key pair kp): keys 2kp, 2kp+1 of each 32-key sub-block
    const int ch = tid & 15, kp = tid >> 4;
    const size_t key_stride = (size_t)Hkv * 128;
    const bf16_t* kbase = k_cache + ((size_t)b * Tmax * Hkv + hk) * 128 + ch * 8;
    const bf16_t* vbase = v_cache + ((size_t)b * Tmax * Hkv + hk) * 128 + ch * 8;
    uint4 rk[2][2], rv[2][2];
    auto fetch = [&](int kb) {
#pragma unroll
        for (int sb = 0; sb < 2; sb++)
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int key = kb + 32 * sb + 2 * kp + i;
                const bool ok = key <= k_hi;
                rk[sb][i] = ok ? *(const uint4*)(kbase + (size_t)key * key_stride) : make_uint4(0, 0, 0, 0);
                rv[sb][i] = ok ? *(const uint4*)(vbase + (size_t)key * key_stride) : make_uint4(0, 0, 0, 0);
            }
    };
    auto stage = [&]() {
#pragma unroll
        for (int sb = 0; sb < 2; sb++) {
#pragma unroll
            for (int i = 0; i < 2; i++) *(uint4*)(lds_k[sb] + (2 * kp + i) * PF_KPITCH + ch * 16) = rk[sb][i];
            // V^T[d = 8ch + e][keys 2kp, 2kp+1] as one dword per e
            const uint32_t a[4] = {rv[sb][0].x, rv[sb][0].y, rv[sb][0].z, rv[sb][0].w}, c[4] = {rv[sb][1].x, rv[sb][1].y, rv[sb][1].z, rv[sb][1].w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const uint32_t lo = (e & 1) ? (a[e >> 1] >> 16) : (a[e >> 1] & 0xffffu);
                const uint32_t hi = (e & 1) ? (c[e >> 1] >> 16) : (c[e >> 1] & 0xffffu);
                *(uint32_t*)(lds_v[sb] + (8 * ch + e) * PF_VPITCH + 4 * kp) = lo | (hi << 16);
            }
        }
    };
    // one sub-block of 32 keys starting at kb, staged in slot sb
    auto sub_block = [&](int kb, int sb) {
        // ---- S^T = K . Q^T : rows = keys kb + 8*(r/4) + 4*hl + r%4, column = this lane's query
        v16f s;
#pragma unroll
        for (int r = 0; r < 16; r++) s[r] = 0.f;
#pragma unroll
        for (int c = 0; c < 8; c++) {
            const v8bf kf = as_v8bf(*(const uint4*)(lds_k[sb] + col * PF_KPITCH + (16 * c + 8 * hl) * 2));
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[c], s, 0, 0, 0);
        }
        // ---- mask, online softmax (per lane = per query; the other half of the keys sits in lane ^ 32)
        float mx = PF_NEG;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const int key = kb + 8 * (r >> 2) + 4 * hl + (r & 3);
            const bool vis = key <= qpos && key >= q_lo && key <= k_hi;
            s[r] = vis ? s[r] * sc : PF_NEG;
            mx = fmaxf(mx, s[r]);
        }
        mx = fmaxf(mx, __shfl_xor(mx, 32));
        const float m_new = fmaxf(m_run, mx);
        const float corr = exp2f(m_run - m_new);
        m_run = m_new;
        float psum = 0.f;
        v8bf pf[2];
#pragma unroll
        for (int r = 0; r < 16; r++) {
            // a fully masked block leaves m_new at PF_NEG: exp2f(0) would be 1, so masked entries are zeroed explicitly
            const float p = s[r] > 0.5f * PF_NEG ? exp2f(s[r] - m_new) : 0.f;
            psum += p;
            pf[r >> 3][r & 7] = (__bf16)p;
        }
        l_run = l_run * corr + psum;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int r = 0; r < 16; r++) o[dt][r] *= corr;
        // ---- O^T += V^T . P^T : chunk c2 of 16 keys uses accumulator rows 8*c2 .. 8*c2+7, i.e. keys
        //      kb + 16*c2 + 4*hl + {0..3} and kb + 16*c2 + 8 + 4*hl + {0..3}; V^T is read in the same order
#pragma unroll
        for (int c2 = 0; c2 < 2; c2++)
#pragma unroll
            for (int dt = 0; dt < 4; dt++) {
                const uint8_t* vrow = lds_v[sb] + (32 * dt + col) * PF_VPITCH + (16 * c2 + 4 * hl) * 2;
                const uint2 lo = *(const uint2*)vrow, hi = *(const uint2*)(vrow + 16);
                const v8bf vf = as_v8bf(make_uint4(lo.x, lo.y, hi.x, hi.y));
                o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pf[c2], o[dt], 0, 0, 0);
            }
    };

    if (kb_first <= k_hi) fetch(kb_first);
    for (int kb = kb_first; kb <= k_hi; kb += 64) {
        __syncthreads();                    // everyone is done with the previous block's tiles
        stage();
        __syncthreads();
        if (kb + 64 <= k_hi) fetch(kb + 64);
        // (wave-uniform tests: a skipped sub-block holds no key that any query of this wave sees)
        if (kb <= w_hi && kb + 31 >= w_lo) sub_block(kb, 0);
        if (kb + 32 <= w_hi && kb + 63 >= w_lo) sub_block(kb + 32, 1);
    }

    // ---- finish: total weight of the query = both lane halves
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv_l = l_tot > 0.f ? 1.0f / l_tot : 0.f;
    float am = 0.f;
    if (q_ok) {
        bf16_t* orow = out + (((size_t)b * T + t) * H + h) * 128;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g4 = 0; g4 < 4; g4++) {
                const int d = 32 * dt + 8 * g4 + 4 * hl;
                const uint2 pk = make_uint2(pack_bf16(o[dt][4 * g4] * inv_l, o[dt][4 * g4 + 1] * inv_l),
                                            pack_bf16(o[dt][4 * g4 + 2] * inv_l, o[dt][4 * g4 + 3] * inv_l));
                *(uint2*)(orow + d) = pk;
                am = fmaxf(am, fmaxf(fmaxf(fabsf(bf16_lo(pk.x)), fabsf(bf16_hi(pk.x))), fmaxf(fabsf(bf16_lo(pk.y)), fabsf(bf16_hi(pk.y)))));
            }
    }
    if (amax_ws) {
        am = wave_max(am);
        __syncthreads();
        if (lane == 0) red[wave] = am;
        __syncthreads();
        if (tid == 0) amax_publish(amax_ws, fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3])));
    }
}

int nc_launch_attention_prefill(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens,
                                int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                                uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(q && k_cache && v_cache && cache_seqlens && out, "prefill_attention: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0 && Hkv > 0 && Tmax > 0 && H % Hkv == 0, "prefill_attention: bad shape");
    NC_CHECK_ARG(B <= 65535 && H <= 65535, "prefill_attention: more than 65535 rows or heads in one launch");
    NC_CHECK_ARG((((uintptr_t)q | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)out) & 15) == 0,
                 "prefill_attention: pointers must be 16-byte aligned");
    NcProfScope prof(0, 0.0, s);
    const int G = H / Hkv;
    const int GS = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);       // query heads of a kv head per workgroup
    const int QT = 128 / GS;
    const dim3 grid((T + QT - 1) / QT, Hkv * (G / GS), B);
    NC_CHECK_ARG(grid.y <= 65535, "prefill_attention: too many heads in one launch");
#define PF_LAUNCH(GG)                                                                                                                  \
    hipLaunchKernelGGL(attn_prefill_kernel<GG>, grid, dim3(256), 0, s, q, k_cache, v_cache, cache_seqlens, window_left, seqlens_include_new, \
                       out, amax_ws, T, H, Hkv, Tmax)
    if (GS == 4) PF_LAUNCH(4);
    else if (GS == 2) PF_LAUNCH(2);
    else PF_LAUNCH(1);
#undef PF_LAUNCH
    NC_CHECK_LAUNCH("prefill_attention");
    return 0;
}
