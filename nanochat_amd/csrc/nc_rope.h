// One head of the q|k|v post-processing of CausalSelfAttention.forward (nanochat/gpt.py:89-104), done by one wave:
// lane L holds elements L and L+64 of the 128-wide head, which is exactly one rotary pair.
//   q and k heads: rotary by the position's angle -> rms_norm over the head -> * 1.2
//   v heads:       v + 3*sigmoid(W_g . xn[:12])[head] * ve[token id, head, :]   (layers with a value embedding)
// Every value is rounded to bf16 wherever the eager bf16 graph of the reference materialises a tensor.
// Shared by the stand-alone rotary/append kernel and by the decode attention kernel that does this work itself.
#pragma once
#include "nc_common.h"
#include "nc_kernels.h"

#define RMS_EPS 1.1920928955078125e-07f   // fp32 machine epsilon: F.rms_norm's default eps

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

struct NcRopeSrc {
    const bf16_t* qkv;        // bf16 [tokens, ld_qkv] output of the q|k|v linear, or nullptr when it is still in partials
    int ld_qkv;
    NcPartialSrc pq;
    const bf16_t* xn;         // normalised layer input (the value-embedding gate reads its first 12 channels)
    int ld_xn;
    const int64_t* idx;       // token ids
    const bf16_t* ve_table;   // nullptr: layer without value embedding
    const float* ve_gate_w;
    const bf16_t* cos_t;
    const bf16_t* sin_t;
    int rope_len;
    int vocab_rows;
    const bf16_t* k_new;      // only for the attention kernel's plain-append form: finished new keys / values [tokens, Hkv, 128]
    const bf16_t* v_new;
};

// The loads of one head, issued in one go so that their latency is paid once and a caller can put other loads behind them:
// the first PRE split partials (or the bf16 value), the rotary pair or the value-embedding pair, and for a value head the
// twelve gate inputs (lane c < 12 holds channel c).
template <int PRE>
struct RopeRaw {
    // exactly what the loads returned: a conversion at load time would make the loading code wait for the value
    float t1[PRE], t2[PRE];   // partial sums; without partials t1[0], t2[0] hold the two bf16 values as loaded (bits in the low half)
    uint32_t e1, e2;          // q, k heads: cos, sin;  v heads with a value embedding: ve[lane], ve[lane + 64]   (bf16 bits)
    uint32_t xg;              // v heads: xn[lane] for lane < 12   (bf16 bits)
    float inv_b;              // partials: inverse weight scale of the head's segment
};

// hh in [0, H): query head; [H, H+Hkv): key head; [H+Hkv, H+2Hkv): value head.
template <int PRE>
__device__ __forceinline__ void rope_head_load(const NcRopeSrc& r, int token, int pos, int hh, int H, int Hkv, int lane, RopeRaw<PRE>& w) {
    // every field gets a value before the first load is issued (a store to a register that may hold a pending load makes the
    // compiler wait for the load; an unset field sends the whole struct to scratch memory)
    w.e1 = w.e2 = w.xg = 0u;
    w.inv_b = 0.f;
#pragma unroll
    for (int u = 0; u < PRE; u++) w.t1[u] = w.t2[u] = 0.f;
    if (r.pq.parts) {
        const float* pp = r.pq.parts + (size_t)token * r.pq.ld + hh * 128 + lane;
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            const size_t o = (size_t)(u < r.pq.nsplit ? u : 0) * r.pq.split_stride;
            w.t1[u] = pp[o], w.t2[u] = pp[o + 64];
        }
        // q | k | v segments end on head boundaries, so the head decides the segment
        w.inv_b = r.pq.inv_b[hh * 128 >= r.pq.seg_end1 ? 2 : (hh * 128 >= r.pq.seg_end0 ? 1 : 0)];
    } else {
        const bf16_t* src = r.qkv + (size_t)token * r.ld_qkv + (size_t)hh * 128;
        w.t1[0] = __uint_as_float((uint32_t)src[lane]), w.t2[0] = __uint_as_float((uint32_t)src[lane + 64]);
    }
    if (hh < H + Hkv) {
        const int rp = pos < r.rope_len ? (pos < 0 ? 0 : pos) : r.rope_len - 1;
        w.e1 = r.cos_t[(size_t)rp * 64 + lane], w.e2 = r.sin_t[(size_t)rp * 64 + lane];
        w.xg = r.cos_t[lane];      // never read for a q or k head; loaded so that xg is the result of a load on every path (see above)
    } else if (r.ve_table) {
        const int hv = hh - H - Hkv;
        int64_t tok = r.idx[token];
        if (tok < 0 || tok >= r.vocab_rows) tok = 0;
        const bf16_t* ve = r.ve_table + ((size_t)tok * Hkv + hv) * 128;
        w.e1 = ve[lane], w.e2 = ve[lane + 64];
        w.xg = r.xn[(size_t)token * r.ld_xn + (lane < 12 ? lane : 0)];
    }
}

// Returns the finished pair.
template <int PRE>
__device__ __forceinline__ void rope_head_finish(const NcRopeSrc& r, int token, int hh, int H, int Hkv, int lane, const RopeRaw<PRE>& w,
                                                 float a_amax /* amax of the linear's input (the word(s) r.pq.a_amax names), read by the caller; used with partials only */, float& o1,
                                                 float& o2) {
    // The conversions below must stay here: moved up to the loads (the compiler does that when it merges the branches of the load
    // step) they would make the loading code wait.  An empty asm that "rewrites" the raw values pins their first use to this point.
    uint32_t e1 = w.e1, e2 = w.e2, xg = w.xg;
    float t10 = w.t1[0], t20 = w.t2[0];
    asm volatile("" : "+v"(e1), "+v"(e2), "+v"(xg), "+v"(t10), "+v"(t20)::"memory");
    float x1, x2;
    if (r.pq.parts) {
        // the linear's output still sits in split partials: add them up in split order, scale, round to bf16
        const int col = hh * 128 + lane;
        float a1 = 0.f, a2 = 0.f;
#pragma unroll
        for (int u = 0; u < PRE; u++)
            if (u < r.pq.nsplit) a1 += u ? w.t1[u] : t10, a2 += u ? w.t2[u] : t20;
        // splits beyond the first PRE, eight at a time, loads first, sums after (see mix_norm_vec_kernel)
        const float* pp = r.pq.parts + (size_t)token * r.pq.ld + col;
        for (int sp0 = PRE; sp0 < r.pq.nsplit; sp0 += 8) {
            float t1[8], t2[8];
#pragma unroll
            for (int u = 0; u < 8; u++) {
                const size_t o = (size_t)(sp0 + u < r.pq.nsplit ? sp0 + u : sp0) * r.pq.split_stride;
                t1[u] = pp[o], t2[u] = pp[o + 64];
            }
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (sp0 + u < r.pq.nsplit) a1 += t1[u], a2 += t2[u];
        }
        const float inv_a = 1.0f / scale_from_amax(a_amax);
        x1 = rbf((a1 * inv_a) * w.inv_b);
        x2 = rbf((a2 * inv_a) * w.inv_b);
    } else {
        x1 = bf16_to_f32((bf16_t)__float_as_uint(t10)), x2 = bf16_to_f32((bf16_t)__float_as_uint(t20));
    }
    if (hh < H + Hkv) {
        const float c = bf16_to_f32((bf16_t)e1), s = bf16_to_f32((bf16_t)e2);
        float y1 = rbf(rbf(x1 * c) + rbf(x2 * s));
        float y2 = rbf(rbf(x1 * (-s)) + rbf(x2 * c));
        const float ss = wave_sum(y1 * y1 + y2 * y2);
        const float rstd = 1.0f / sqrtf(ss / 128.0f + RMS_EPS);
        o1 = rbf(rbf(y1 * rstd) * 1.2f);
        o2 = rbf(rbf(y2 * rstd) * 1.2f);
    } else {
        const int hv = hh - H - Hkv;
        if (r.ve_table) {
            float dot = 0.f;
#pragma unroll
            for (int cidx = 0; cidx < 12; cidx++)
                dot += bf16_to_f32((bf16_t)__builtin_amdgcn_readlane((int)xg, cidx)) * rbf(r.ve_gate_w[hv * 12 + cidx]);
            const float gate = rbf(3.0f * rbf(sigmoidf_(rbf(dot))));
            x1 = rbf(x1 + rbf(gate * bf16_to_f32((bf16_t)e1)));
            x2 = rbf(x2 + rbf(gate * bf16_to_f32((bf16_t)e2)));
        }
        o1 = x1, o2 = x2;
    }
}

__device__ __forceinline__ void rope_head(const NcRopeSrc& r, int token, int pos, int hh, int H, int Hkv, int lane, float& o1, float& o2) {
    RopeRaw<8> w;
    const uint32_t amax_lane = r.pq.parts ? amax_load_lane(r.pq.a_amax) : 0u;
    rope_head_load(r, token, pos, hh, H, Hkv, lane, w);
    rope_head_finish(r, token, hh, H, Hkv, lane, w, amax_from_lanes(amax_lane), o1, o2);
}
