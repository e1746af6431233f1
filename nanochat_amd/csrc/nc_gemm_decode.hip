// Small-M (decode) FP8 linear:  out[M,N] = epilogue((A[M,K] . W[N,K]^T, fp32 acc) * inv_a * inv_w),  M <= 128.
// This is Float8Linear.forward (nanochat/fp8.py:202-213) at decode time, where the weight stream from HBM is
// the whole cost: N*K bytes of e4m3 per call against M*K of activations.
//
// Work split: a workgroup (4 waves) owns 64 output columns (16 per wave) and a range of K-steps (128
// wide); grid = (N/64) x ksplits so that even a 1664x1664 weight (2.8 MB) is spread over a few hundred
// workgroups and every CU pulls a few KB.  Weight rows go global -> registers (one 16x128-byte MFMA
// fragment per wave per K-step, two 16-byte loads per lane, rows contiguous).  The activation panel of
// the K range is shared by the 4 waves through LDS; when A arrives as bf16 plus its tensorwise amax, it is
// quantized to e4m3 on the way into LDS (scale = fp32(448/max(fp64(amax),1e-12)), saturate, RNE), so the
// separate convert pass of the quantizer disappears.
//
// A dependent trip to memory costs a couple of microseconds here, which is more than the arithmetic of one of
// these GEMMs, so the kernels are built to make as few as they can, and with split-K the raw fp32 partial tiles
// are simply stored ([split][M][N]) -- the kernel that consumes the linear's output (residual/norm,
// rotary/append, or nc_finish_partials) adds the splits in a fixed order, applies inv_a * inv_w and rounds to
// bf16 while it reads them, which it had to read anyway.  Three forms:
//   gemm_decode_onetrip_kernel  a K range of at most 8 steps per workgroup (every split linear of a decode step):
//                               the whole range asked for through buffer descriptors before the first wait
//                               (9.0 / 6.7 / 9.9 / 9.7 us -> 8.2 / 5.0 / 8.3 / 8.5 us for the four linears of a
//                               d26 layer at 64 rows; about 3.4 us of each is the weight fetch itself, 2.3 us the
//                               launch, 1.5 us the partial sums leaving the chip); 65 .. 128 rows take eight
//                               waves, two halves of 64 rows against the same weight columns (d26 at 128 rows
//                               with the prompt read once: 39.7 k -> 43.1 k tokens/s);
//   gemm_decode_full_kernel     17 .. 64 rows, K <= 2048, relu^2 epilogue: unsplit, 32 columns per workgroup,
//                               the result leaves finished and the MLP activation needs no pass of its own
//                               (10.6 us against 8.3 + 4.4 us for the split linear and its finishing pass);
//   gemm_decode_kernel          everything else (longer K ranges walked in 512-wide chunks).
//
// Epilogues: 0 bf16;  1 fp32 softcap*tanh(bf16(v)/softcap) (lm_head, nanochat/gpt.py:512-515);
//            2 bf16 relu(bf16(v))^2 plus atomic amax of the result (MLP activation, gpt.py:139).
#include <hip/hip_ext.h>
#include "nc_common.h"
#include "nc_kernels.h"
#include "nc_rope.h"

#define MFMA_F8(acc, b, a) __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4((b), (a), (acc), 0, 0, 0, 0, 0, 0)

struct DecodeGemmArgs {
    const void* A;            // e4m3 [M,K] or bf16 [M,K]
    const uint32_t* a_amax;   // bf16 mode: fp32 bits of max|A|
    const float* inv_a;       // e4m3 mode: inverse scale of A
    const uint8_t* B;
    const float* inv_b;
    NcGemmSegs segs;
    void* out;
    int out_kind;
    float softcap;
    int ldc;
    uint32_t* out_amax;       // out_kind 2
    float* partial_out;       // ksplits > 1: [ksplits][M][N] raw fp32 sums
    int ksplits, ksteps_per_split;
    int M, N, K;
    NcRowRecipe recipe;       // A_MODE 2
};

__device__ __forceinline__ float dg_seg_scale(const DecodeGemmArgs& g, int col) {
    int s = 0;
#pragma unroll
    for (int i = 0; i < 3; i++)
        if (i + 1 < g.segs.nseg && col >= g.segs.end[i]) s = i + 1;
    return g.inv_b[s];
}

// The rows of A from a recipe, as bf16 in `rowbuf` ([M][K]); returns their amax.  Thread t owns elements 8t .. 8t+7 (+2048 per further
// pass) of a row, the mapping of mix_norm_vec_kernel, and every sum runs in that kernel's order.  Everything a row needs is asked for
// before anything is waited for (the work is a trip to memory and two reductions; the trips are what it costs).
template <int KIND>
__device__ __forceinline__ float recipe_rows(const NcRowRecipe& r, bf16_t* rowbuf, float* red, int M, int K, bool writer) {
    const int tid = threadIdx.x;
    const bool has_parts = r.padd.parts != nullptr;
    const uint32_t p_amax_lane = has_parts ? amax_load_lane(r.padd.a_amax) : 0u;
    const float p_inv_b = has_parts ? r.padd.inv_b[0] : 0.f;
    float am = 0.f;
    if (KIND == 1) {
        const float rl_raw = r.resid_lambda ? *r.resid_lambda : 0.f, xl_raw = r.x0_lambda ? *r.x0_lambda : 0.f;
        const int c = tid * 8;
        const bool live = c < K;                     // K <= 2048: one pass
        for (int m = 0; m < M; m++) {
            const size_t at = (size_t)m * K + (live ? c : 0);
            uint4 xv = make_uint4(0, 0, 0, 0), av = xv, zv = xv;
            float4 a0[8], a1[8];
            if (live) {
                xv = *(const uint4*)(r.x_in + at);
                if (r.add) av = *(const uint4*)(r.add + at);
                if (r.resid_lambda) zv = *(const uint4*)(r.x0 + at);
                if (has_parts) {
                    const float* pp = r.padd.parts + (size_t)m * r.padd.ld + c;
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const float* q = pp + (size_t)(u < r.padd.nsplit ? u : 0) * r.padd.split_stride;
                        a0[u] = *(const float4*)q;
                        a1[u] = *(const float4*)(q + 4);
                    }
                }
            }
            const float p_inv_a = has_parts ? 1.0f / scale_from_amax(amax_from_lanes(p_amax_lane)) : 0.f;
            const float rl = rbf(rl_raw), xl = rbf(xl_raw);
            float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            float ss = 0.f;
            if (live) {
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
                for (int j = 0; j < 4; j++) v[2 * j] = bf16_lo(xw[j]), v[2 * j + 1] = bf16_hi(xw[j]);
                if (r.add) {
                    const uint32_t aw[4] = {av.x, av.y, av.z, av.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        v[2 * j] = rbf(v[2 * j] + bf16_lo(aw[j]));
                        v[2 * j + 1] = rbf(v[2 * j + 1] + bf16_hi(aw[j]));
                    }
                }
                if (has_parts) {
                    float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        if (u < r.padd.nsplit) {
                            acc8[0] += a0[u].x, acc8[1] += a0[u].y, acc8[2] += a0[u].z, acc8[3] += a0[u].w;
                            acc8[4] += a1[u].x, acc8[5] += a1[u].y, acc8[6] += a1[u].z, acc8[7] += a1[u].w;
                        }
                    }
                    const float* pp = r.padd.parts + (size_t)m * r.padd.ld + c;
                    for (int sp0 = 8; sp0 < r.padd.nsplit; sp0 += 8) {
                        float4 b0[8], b1[8];
#pragma unroll
                        for (int u = 0; u < 8; u++) {
                            const float* q = pp + (size_t)(sp0 + u < r.padd.nsplit ? sp0 + u : sp0) * r.padd.split_stride;
                            b0[u] = *(const float4*)q;
                            b1[u] = *(const float4*)(q + 4);
                        }
#pragma unroll
                        for (int u = 0; u < 8; u++) {
                            if (sp0 + u < r.padd.nsplit) {
                                acc8[0] += b0[u].x, acc8[1] += b0[u].y, acc8[2] += b0[u].z, acc8[3] += b0[u].w;
                                acc8[4] += b1[u].x, acc8[5] += b1[u].y, acc8[6] += b1[u].z, acc8[7] += b1[u].w;
                            }
                        }
                    }
#pragma unroll
                    for (int j = 0; j < 8; j++) v[j] = rbf(v[j] + rbf((acc8[j] * p_inv_a) * p_inv_b));
                }
                if (r.save && writer)
                    *(uint4*)(r.save + at) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
                if (r.resid_lambda) {
                    const uint32_t zw[4] = {zv.x, zv.y, zv.z, zv.w};
#pragma unroll
                    for (int j = 0; j < 4; j++) {
                        v[2 * j] = rbf(rbf(rl * v[2 * j]) + rbf(xl * bf16_lo(zw[j])));
                        v[2 * j + 1] = rbf(rbf(rl * v[2 * j + 1]) + rbf(xl * bf16_hi(zw[j])));
                    }
                }
                if (writer)
                    *(uint4*)(r.x_out + at) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
#pragma unroll
                for (int j = 0; j < 8; j++) ss += v[j] * v[j];
            }
            ss = block_sum<4>(ss, red);
            const float rstd = 1.0f / sqrtf(ss / (float)K + RMS_EPS);
            if (live) {
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    o[j] = pack_bf16(v[2 * j] * rstd, v[2 * j + 1] * rstd);
                    am = amax_fold(amax_fold(am, bf16_lo(o[j])), bf16_hi(o[j]));
                }
                const uint4 ov = make_uint4(o[0], o[1], o[2], o[3]);
                *(uint4*)(rowbuf + (size_t)m * K + c) = ov;
                if (writer && r.xn_out) *(uint4*)(r.xn_out + (size_t)m * K + c) = ov;
            }
        }
    } else {
        // at most four passes of 2048 elements per row (K <= 8192); the partial sums of all of them are asked for at once when the
        // linear was split in two (the c_fc of a decode step), else pass by pass
        const bool two = r.padd.nsplit == 2;
        for (int m = 0; m < M; m++) {
            const float* pp = r.padd.parts + (size_t)m * r.padd.ld;
            float4 q0[4][2], q1[4][2];
            if (two) {
#pragma unroll
                for (int ps = 0; ps < 4; ps++) {
                    const int c = tid * 8 + 2048 * ps;
                    const float* q = pp + (c < K ? c : 0);
                    q0[ps][0] = *(const float4*)q, q1[ps][0] = *(const float4*)(q + 4);
                    q0[ps][1] = *(const float4*)(q + r.padd.split_stride), q1[ps][1] = *(const float4*)(q + r.padd.split_stride + 4);
                }
            }
            const float p_inv_a = 1.0f / scale_from_amax(amax_from_lanes(p_amax_lane));
#pragma unroll
            for (int ps = 0; ps < 4; ps++) {
                const int c = tid * 8 + 2048 * ps;
                if (c < K) {
                    float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                    if (two) {
#pragma unroll
                        for (int u = 0; u < 2; u++) {
                            acc8[0] += q0[ps][u].x, acc8[1] += q0[ps][u].y, acc8[2] += q0[ps][u].z, acc8[3] += q0[ps][u].w;
                            acc8[4] += q1[ps][u].x, acc8[5] += q1[ps][u].y, acc8[6] += q1[ps][u].z, acc8[7] += q1[ps][u].w;
                        }
                    } else {
                        for (int sp = 0; sp < r.padd.nsplit; sp++) {
                            const float* q = pp + (size_t)sp * r.padd.split_stride + c;
                            const float4 b0 = *(const float4*)q, b1 = *(const float4*)(q + 4);
                            acc8[0] += b0.x, acc8[1] += b0.y, acc8[2] += b0.z, acc8[3] += b0.w;
                            acc8[4] += b1.x, acc8[5] += b1.y, acc8[6] += b1.z, acc8[7] += b1.w;
                        }
                    }
                    float h[8];
#pragma unroll
                    for (int j = 0; j < 8; j++) {
                        const float t = relu_keep_nan(rbf((acc8[j] * p_inv_a) * p_inv_b));
                        h[j] = rbf(t * t);
                        am = amax_join(am, h[j]);
                    }
                    *(uint4*)(rowbuf + (size_t)m * K + c) = make_uint4(pack_bf16(h[0], h[1]), pack_bf16(h[2], h[3]), pack_bf16(h[4], h[5]), pack_bf16(h[6], h[7]));
                }
            }
        }
    }
    am = wave_amax(am);
    __syncthreads();
    if ((tid & 63) == 0) red[tid >> 6] = am;
    __syncthreads();
    am = amax_join(amax_join(red[0], red[1]), amax_join(red[2], red[3]));
    if (writer && tid == 0) amax_publish(r.amax_out, am);
    __syncthreads();                                   // the rows are complete in LDS, `red` is free again
    return am;
}

// A_MODE 0: A is e4m3 with its inverse scale; 1: bf16 with the amax word of its producer; 2 / 3: made by the kernel from a recipe of
// kind 1 / 2.
template <int MB, int A_MODE>
__global__ __launch_bounds__(256) void gemm_decode_kernel(DecodeGemmArgs g) {
    constexpr bool A_BF16 = A_MODE != 0;
    constexpr int ROWS = MB * 16;
    constexpr int A_CH = ROWS * 32 / 256;          // 16-byte LDS chunks per thread per 512-wide sub-chunk
    __shared__ __align__(16) uint8_t lds[2][ROWS * 512];
    __shared__ float red[8];
    __shared__ __align__(16) bf16_t rowbuf[A_MODE == 2 ? NC_RECIPE_MAX_ROWS * 2048 : (A_MODE == 3 ? NC_RECIPE_MAX_ROWS * NC_RECIPE_MAX_K : 8)];

    NC_ARG_NOW(g.A); NC_ARG_NOW(g.a_amax); NC_ARG_NOW(g.inv_a); NC_ARG_NOW(g.B); NC_ARG_NOW(g.partial_out); NC_ARG_NOW(g.ksplits);
    NC_ARG_NOW(g.ksteps_per_split); NC_ARG_NOW(g.M); NC_ARG_NOW(g.N); NC_ARG_NOW(g.K);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int frow = lane & 15, kb = lane >> 4;
    const int nblk = blockIdx.x, split = blockIdx.y;
    const int M = g.M, N = g.N, K = g.K;
    const int n0 = nblk * 64 + wave * 16;
    const int brow = n0 + frow;
    const bool brow_ok = brow < N;
    const uint8_t* bptr = g.B + (size_t)(brow_ok ? brow : 0) * K + kb * 32;

    const int nksteps = (K + 127) >> 7;
    const int ks_begin = split * g.ksteps_per_split;
    int ks_end = ks_begin + g.ksteps_per_split;
    if (ks_end > nksteps) ks_end = nksteps;
    const int k_hi = (ks_end << 7) < K ? (ks_end << 7) : K;       // exclusive K bound of this split

    // the activation scale is asked for here and looked at only after the first operand loads are on their way
    const uint32_t amax_lane = A_MODE == 1 ? amax_load_lane(g.a_amax) : 0u;
    float scale = 1.f, inv_a = A_BF16 ? 0.f : *g.inv_a;

    v4f acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};

    uint4 ra[A_CH][A_BF16 ? 2 : 1];
    uint4 rb[2][4][2];
    // sub-chunk c covers K-steps [ks_begin + 4c, ks_begin + 4c + 4)
    auto load_a = [&](int k0) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 5, ch = id & 31;
            const int gk = k0 + ch * 16;
            const bool ok = row < M && gk < k_hi;
            if (A_MODE >= 2) {
                const uint4* p = (const uint4*)(rowbuf + (ok ? (size_t)row * K + gk : 0));
                ra[c][0] = ok ? p[0] : make_uint4(0, 0, 0, 0);
                ra[c][A_BF16 ? 1 : 0] = ok ? p[1] : make_uint4(0, 0, 0, 0);
            } else if (A_BF16) {
                const uint4* p = (const uint4*)((const bf16_t*)g.A + (size_t)row * K + gk);
                ra[c][0] = ok ? p[0] : make_uint4(0, 0, 0, 0);
                ra[c][A_BF16 ? 1 : 0] = ok ? p[1] : make_uint4(0, 0, 0, 0);
            } else {
                ra[c][0] = ok ? *(const uint4*)((const uint8_t*)g.A + (size_t)row * K + gk) : make_uint4(0, 0, 0, 0);
            }
        }
    };
    auto store_a = [&](int buf) {
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * 256, row = id >> 5, ch = id & 31;
            uint4 v;
            if (A_BF16) {
                const uint32_t w[8] = {ra[c][0].x, ra[c][0].y, ra[c][0].z, ra[c][0].w,
                                       ra[c][A_BF16 ? 1 : 0].x, ra[c][A_BF16 ? 1 : 0].y, ra[c][A_BF16 ? 1 : 0].z, ra[c][A_BF16 ? 1 : 0].w};
                uint32_t o[4];
#pragma unroll
                for (int j = 0; j < 4; j++)
                    // no clamp needed: |x| <= amax gives |x*scale| <= 448*(1+2^-23), which rounds to 448 like the clamped value
                    o[j] = e4m3_pack4_hw(bf16_lo(w[2 * j]) * scale, bf16_hi(w[2 * j]) * scale, bf16_lo(w[2 * j + 1]) * scale,
                                         bf16_hi(w[2 * j + 1]) * scale);
                v = make_uint4(o[0], o[1], o[2], o[3]);
            } else {
                v = ra[c][0];
            }
            *(uint4*)(&lds[buf][row * 512 + ((ch ^ (row & 15)) << 4)]) = v;
        }
    };
    auto load_b = [&](int k0, int slot) {
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            const int gk = k0 + kk * 128 + kb * 32;
#pragma unroll
            for (int h = 0; h < 2; h++)
                rb[slot][kk][h] = (brow_ok && gk + h * 16 < k_hi) ? *(const uint4*)(bptr + k0 + kk * 128 + h * 16)
                                                                 : make_uint4(0, 0, 0, 0);
        }
    };

    const int nsub = (ks_end - ks_begin + 3) >> 2;
    const int kbase = ks_begin << 7;
    auto compute = [&](int s, int buf, int slot) {
        const int nk = min(4, ks_end - ks_begin - 4 * s);
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            if (kk < nk) {
                v8i bf;
                const uint4 lo = rb[slot][kk][0], hi = rb[slot][kk][1];
                bf[0] = lo.x, bf[1] = lo.y, bf[2] = lo.z, bf[3] = lo.w, bf[4] = hi.x, bf[5] = hi.y, bf[6] = hi.z, bf[7] = hi.w;
#pragma unroll
                for (int i = 0; i < MB; i++) {
                    const int row = i * 16 + frow;
                    const int c0 = kk * 8 + 2 * kb;
                    const uint4 alo = *(const uint4*)(&lds[buf][row * 512 + ((c0 ^ (row & 15)) << 4)]);
                    const uint4 ahi = *(const uint4*)(&lds[buf][row * 512 + (((c0 + 1) ^ (row & 15)) << 4)]);
                    v8i af;
                    af[0] = alo.x, af[1] = alo.y, af[2] = alo.z, af[3] = alo.w, af[4] = ahi.x, af[5] = ahi.y, af[6] = ahi.z, af[7] = ahi.w;
                    acc[i] = MFMA_F8(acc[i], bf, af);
                }
            }
        }
    };
    {
        if (nsub > 0) load_b(kbase, 0);
        if (A_MODE >= 2) {
            // the weights are on their way while the rows are made
            scale = scale_from_amax(recipe_rows<A_MODE - 1>(g.recipe, rowbuf, red, M, K, blockIdx.x == 0 && blockIdx.y == 0));
            inv_a = 1.0f / scale;
        }
        if (nsub > 0) load_a(kbase);
        if (A_MODE == 1) {
            scale = scale_from_amax(amax_from_lanes(amax_lane));
            inv_a = 1.0f / scale;
        }
        if (nsub > 0) store_a(0);
        __syncthreads();
#pragma unroll 1
        for (int sc = 0; sc < nsub; sc += 2) {
#pragma unroll
            for (int half = 0; half < 2; half++) {
                const int s = sc + half;
                if (s < nsub) {
                    const bool more = s + 1 < nsub;
                    if (more) {
                        load_b(kbase + (s + 1) * 512, half ^ 1);
                        load_a(kbase + (s + 1) * 512);
                    }
                    compute(s, half, half);
                    if (more) store_a(half ^ 1);
                    __syncthreads();
                }
            }
        }
    }

    // ---- split-K: store the raw partial tile; the consumer adds the splits
    if (g.ksplits > 1) {
        const int n = n0 + 4 * kb;
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const int m = i * 16 + frow;
            if (m < M && n < N)
                *(float4*)(g.partial_out + ((size_t)split * M + m) * N + n) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
        }
        return;
    }

    // ---- epilogue: lane holds rows i*16 + frow, columns n0 + 4*kb .. +3
    float am = 0.f;
    const int n = n0 + 4 * kb;
#pragma unroll
    for (int i = 0; i < MB; i++) {
        const int m = i * 16 + frow;
        if (m < M && n < N) {
            const float inv_b = dg_seg_scale(g, n);
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = (acc[i][r] * inv_a) * inv_b;
            if (g.out_kind == 1) {
                float* o = (float*)g.out + (size_t)m * g.ldc + n;
                for (int r = 0; r < 4 && n + r < N; r++) o[r] = g.softcap * tanhf(rbf(v[r]) / g.softcap);
            } else {
                if (g.out_kind == 2) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float t = relu_keep_nan(rbf(v[r]));
                        v[r] = rbf(t * t);
                        if (n + r < N) am = amax_join(am, v[r]);
                    }
                }
                bf16_t* o = (bf16_t*)g.out + (size_t)m * g.ldc + n;
                if (n + 3 < N) *(uint2*)o = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
                else
                    for (int r = 0; r < 4 && n + r < N; r++) o[r] = f32_to_bf16(v[r]);
            }
        }
    }
    if (g.out_kind == 2 && g.out_amax) {
        am = wave_amax(am);
        if (lane == 0) red[wave] = am;
        __syncthreads();
        if (tid == 0) {
            am = amax_join(amax_join(red[0], red[1]), amax_join(red[2], red[3]));
            amax_publish(g.out_amax, am);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// The same work when a workgroup's K range is at most 8 steps (every split linear of a decode step): one trip to memory.  All loads
// go through buffer descriptors, whose range check returns zeros for rows past M / N and for whatever lies beyond the K range, so no
// load sits under a branch and the whole range -- activation rows first (they come from the L2 and are converted into LDS while the
// weight rows are still on their way), then the weight rows -- is asked for before anything is waited for.  The tensorwise amax comes
// through the scalar cache, which has a counter of its own.
#define NC_DG_OOB 0x80000000u
typedef int dg_v4i __attribute__((ext_vector_type(4)));
// A_MODE as in gemm_decode_kernel: 0 e4m3 activations, 1 bf16 + the producer's amax, 2 / 3 rows made here from a recipe of kind 1 / 2
// (one or two rows; the weight rows are on their way while the rows are made).
// WR: 1 = four waves, up to 64 rows; 2 = eight waves for 65 .. 128 rows, waves 4 .. 7 multiplying rows 64 .. 127 with the same columns.
// The occupancy is pinned so that the scheduler keeps every load of the range in flight instead of trading them for registers.
template <int MB, int A_MODE, int NSET, int WR = 1>
__global__ __launch_bounds__(256 * WR) __attribute__((amdgpu_waves_per_eu(WR, 2))) void gemm_decode_onetrip_kernel(DecodeGemmArgs g) {
    constexpr bool A_BF16 = A_MODE != 0;
    constexpr int ROWS = MB * 16 * WR, NT = 256 * WR;
    constexpr int A_CH = ROWS * 32 / NT;           // 16-byte e4m3 chunks per thread per 512-wide half of the range
    constexpr int A_LD = A_BF16 ? 2 : 1;
    extern __shared__ __align__(16) uint8_t lds_raw[];             // NSET panels of ROWS x 512 bytes
    uint8_t (*lds)[ROWS * 512] = (uint8_t (*)[ROWS * 512])lds_raw;
    __shared__ float red[8];
    __shared__ __align__(16) bf16_t rowbuf[A_MODE == 2 ? NC_RECIPE_MAX_ROWS * 2048 : (A_MODE == 3 ? NC_RECIPE_MAX_ROWS * NC_RECIPE_MAX_K : 8)];

    NC_ARG_NOW(g.A); NC_ARG_NOW(g.a_amax); NC_ARG_NOW(g.inv_a); NC_ARG_NOW(g.B); NC_ARG_NOW(g.partial_out); NC_ARG_NOW(g.ksplits);
    NC_ARG_NOW(g.ksteps_per_split); NC_ARG_NOW(g.M); NC_ARG_NOW(g.N); NC_ARG_NOW(g.K);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int frow = lane & 15, kb = lane >> 4;
    const int split = blockIdx.y;
    const int M = g.M, N = g.N, K = g.K;
    const int n0 = blockIdx.x * 64 + (wave & 3) * 16;
    const int rbase = (wave >> 2) * MB * 16;                       // first row this wave multiplies
    const int brow = n0 + frow;

    const int nksteps = (K + 127) >> 7;
    const int ks_begin = split * g.ksteps_per_split;
    int ks_end = ks_begin + g.ksteps_per_split;
    if (ks_end > nksteps) ks_end = nksteps;
    const int nk = ks_end - ks_begin;                              // 1 .. 4 * NSET
    const int kbase = ks_begin << 7;
    const int k_hi = (ks_end << 7) < K ? (ks_end << 7) : K;       // exclusive K bound of this split

    AmaxWords aw = {};
    float inv_a = 0.f;
    if (A_MODE == 1) aw = amax_load_scalar(g.a_amax);
    else if (A_MODE == 0) inv_a = *g.inv_a;

    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)g.A, 0, M * K * (A_BF16 ? 2 : 1), 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)g.B, 0, N * K, 0x00020000);

    // (measured: handing the conversion to waves of their own, so that the weight requests go out first, is slower, 9.9 against
    // 8.3 us at N = 6656, K = 1664)
    dg_v4i ra[NSET][A_CH][A_LD], rb[NSET][4][2];
    if (A_MODE < 2) {
#pragma unroll
        for (int set = 0; set < NSET; set++)
#pragma unroll
            for (int c = 0; c < A_CH; c++) {
                const int id = tid + c * NT, row = id >> 5, ch = id & 31;
                const int gk = kbase + set * 512 + ch * 16;
                const uint32_t vo = (row < M && gk < k_hi) ? ((uint32_t)row * (uint32_t)K + (uint32_t)gk) * (A_BF16 ? 2u : 1u) : NC_DG_OOB;
#pragma unroll
                for (int h = 0; h < A_LD; h++) ra[set][c][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_a, vo, h * 16, 0);
            }
    }
#pragma unroll
    for (int set = 0; set < NSET; set++)
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
            // a lane's 32 K-bytes of a step are pieces kb and 4 + kb of its 128 (the activation side reads the same pieces): the four
            // lanes of a row then ask for 64 contiguous bytes per instruction
            const int gk = kbase + set * 512 + kk * 128 + kb * 16;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint32_t vo = (brow < N && gk + h * 64 < k_hi) ? (uint32_t)brow * (uint32_t)K + (uint32_t)gk : NC_DG_OOB;
                rb[set][kk][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_b, vo, h * 64, 0);
            }
        }

    float scale = 1.f;
    if (A_MODE == 1) {
        scale = scale_from_amax(amax_from_words(aw));
        inv_a = 1.0f / scale;
    }
    if (A_MODE >= 2) {
        // the rows from their recipe, as bf16 in LDS, then this workgroup's K range of them into the staging registers
        scale = scale_from_amax(recipe_rows<A_MODE - 1>(g.recipe, rowbuf, red, M, K, blockIdx.x == 0 && blockIdx.y == 0));
        inv_a = 1.0f / scale;
#pragma unroll
        for (int set = 0; set < NSET; set++)
#pragma unroll
            for (int c = 0; c < A_CH; c++) {
                const int id = tid + c * NT, row = id >> 5, ch = id & 31;
                const int gk = kbase + set * 512 + ch * 16;
                const bool ok = row < M && gk < k_hi;
                const dg_v4i* p = (const dg_v4i*)(rowbuf + (ok ? (size_t)row * K + gk : 0));
                const dg_v4i z = {0, 0, 0, 0};
                ra[set][c][0] = ok ? p[0] : z;
                ra[set][c][A_LD - 1] = ok ? p[1] : z;
            }
    }
#pragma unroll
    for (int set = 0; set < NSET; set++)
#pragma unroll
        for (int c = 0; c < A_CH; c++) {
            const int id = tid + c * NT, row = id >> 5, ch = id & 31;
            dg_v4i v;
            if (A_BF16) {
                const uint32_t w[8] = {(uint32_t)ra[set][c][0][0], (uint32_t)ra[set][c][0][1], (uint32_t)ra[set][c][0][2], (uint32_t)ra[set][c][0][3],
                                       (uint32_t)ra[set][c][A_LD - 1][0], (uint32_t)ra[set][c][A_LD - 1][1], (uint32_t)ra[set][c][A_LD - 1][2],
                                       (uint32_t)ra[set][c][A_LD - 1][3]};
#pragma unroll
                for (int j = 0; j < 4; j++)
                    // no clamp needed: |x| <= amax gives |x*scale| <= 448*(1+2^-23), which rounds to 448 like the clamped value
                    v[j] = (int)e4m3_pack4_hw(bf16_lo(w[2 * j]) * scale, bf16_hi(w[2 * j]) * scale, bf16_lo(w[2 * j + 1]) * scale,
                                              bf16_hi(w[2 * j + 1]) * scale);
            } else {
                v = ra[set][c][0];
            }
            *(dg_v4i*)(&lds[set][row * 512 + ((ch ^ (row & 15)) << 4)]) = v;
        }
    __syncthreads();

    v4f acc[MB];
#pragma unroll
    for (int i = 0; i < MB; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    // K-steps in pairs; the steps past the range hold zeros on both sides, so only whole pairs are skipped
#pragma unroll
    for (int pr = 0; pr < 2 * NSET; pr++) {
        if (2 * pr < nk) {
            dg_v4i alo[2][MB], ahi[2][MB];
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int kk = (2 * pr + q) & 3;
#pragma unroll
                for (int i = 0; i < MB; i++) {
                    const int row = rbase + i * 16 + frow;
                    const int c0 = kk * 8 + kb;
                    alo[q][i] = *(const dg_v4i*)(&lds[pr >> 1][row * 512 + ((c0 ^ (row & 15)) << 4)]);
                    ahi[q][i] = *(const dg_v4i*)(&lds[pr >> 1][row * 512 + (((c0 + 4) ^ (row & 15)) << 4)]);
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int q = 0; q < 2; q++) {
                const int kk = (2 * pr + q) & 3;
                const dg_v4i lo = rb[pr >> 1][kk][0], hi = rb[pr >> 1][kk][1];
                v8i bf;
                bf[0] = lo[0], bf[1] = lo[1], bf[2] = lo[2], bf[3] = lo[3], bf[4] = hi[0], bf[5] = hi[1], bf[6] = hi[2], bf[7] = hi[3];
#pragma unroll
                for (int i = 0; i < MB; i++) {
                    v8i af;
                    af[0] = alo[q][i][0], af[1] = alo[q][i][1], af[2] = alo[q][i][2], af[3] = alo[q][i][3];
                    af[4] = ahi[q][i][0], af[5] = ahi[q][i][1], af[6] = ahi[q][i][2], af[7] = ahi[q][i][3];
                    acc[i] = MFMA_F8(acc[i], bf, af);
                }
            }
        }
    }

    const int n = n0 + 4 * kb;
    if (g.ksplits > 1) {
        // split-K: the raw partial tile; the consumer adds the splits
#pragma unroll
        for (int i = 0; i < MB; i++) {
            const int m = rbase + i * 16 + frow;
            if (m < M && n < N)
                *(float4*)(g.partial_out + ((size_t)split * M + m) * N + n) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
        }
        return;
    }
    // one split (K <= 1024): the epilogue of gemm_decode_kernel
    float am = 0.f;
#pragma unroll
    for (int i = 0; i < MB; i++) {
        const int m = rbase + i * 16 + frow;
        if (m < M && n < N) {
            const float inv_b = dg_seg_scale(g, n);
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = (acc[i][r] * inv_a) * inv_b;
            if (g.out_kind == 1) {
                float* o = (float*)g.out + (size_t)m * g.ldc + n;
                for (int r = 0; r < 4 && n + r < N; r++) o[r] = g.softcap * tanhf(rbf(v[r]) / g.softcap);
            } else {
                if (g.out_kind == 2) {
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        const float t = relu_keep_nan(rbf(v[r]));
                        v[r] = rbf(t * t);
                        if (n + r < N) am = amax_join(am, v[r]);
                    }
                }
                bf16_t* o = (bf16_t*)g.out + (size_t)m * g.ldc + n;
                if (n + 3 < N) *(uint2*)o = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
                else
                    for (int r = 0; r < 4 && n + r < N; r++) o[r] = f32_to_bf16(v[r]);
            }
        }
    }
    if (g.out_kind == 2 && g.out_amax) {
        am = wave_amax(am);
        if (lane == 0) red[wave] = am;
        __syncthreads();
        if (tid == 0) {
            am = amax_join(amax_join(red[0], red[1]), amax_join(red[2], red[3]));
            if (WR == 2) am = amax_join(am, amax_join(amax_join(red[4], red[5]), amax_join(red[6], red[7])));
            amax_publish(g.out_amax, am);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Unsplit form for 17 .. 64 rows and K <= 2048 (the q|k|v and c_fc linears of a decode step): a workgroup of 8 waves owns 32 output
// columns over the whole of K, so the result leaves the kernel finished (bf16, relu^2 and its amax included) instead of as fp32
// partial sums that cost more to write and to read back than the weights did, and the MLP activation needs no pass of its own.
// The whole activation panel is converted into LDS once per workgroup ([K-step][64 rows][128 bytes] tiles); wave (cb, rh, kh) then
// multiplies rows 32*rh .. +31 with columns 16*cb .. +15 over half of the K-steps, and the two K halves meet through LDS.
// Still one trip to memory: activation rows first, then the weight rows, everything asked for before the first wait.
#define NC_DGF_MAX_K 2048
template <bool A_BF16, int NKS>
__global__ __launch_bounds__(1024) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_decode_full_kernel(DecodeGemmArgs g) {
    constexpr int A_LD = A_BF16 ? 2 : 1;
    constexpr int NKQ = (NKS + 3) / 4;              // K-steps per quarter
    extern __shared__ __align__(16) uint8_t dgf_lds[];            // NKS tiles of 8 KB, then 6 x 4 KB for the meeting of the quarters
    float* const meet = (float*)(dgf_lds + NKS * 8192);
    __shared__ float red[2];

    NC_ARG_NOW(g.A); NC_ARG_NOW(g.a_amax); NC_ARG_NOW(g.inv_a); NC_ARG_NOW(g.B); NC_ARG_NOW(g.inv_b); NC_ARG_NOW(g.out); NC_ARG_NOW(g.out_kind);
    NC_ARG_NOW(g.out_amax); NC_ARG_NOW(g.ldc); NC_ARG_NOW(g.M); NC_ARG_NOW(g.N); NC_ARG_NOW(g.K);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int M = g.M, N = g.N, K = g.K;
    const int nksteps = (K + 127) >> 7;                            // <= NKS

    AmaxWords aw = {};
    float inv_a = 0.f;
    if (A_BF16) aw = amax_load_scalar(g.a_amax);
    else inv_a = *g.inv_a;

    if (wave >= 8) {
        // ---- the converting waves: thread t converts chunk (row t >> 3, 16-byte piece t & 7) of every K-step tile.  Their loads
        // come from the L2; they are asked for after the scale is known, which lets the weight requests of the other waves, the
        // long trip, through the address units first.
        float scale = 1.f;
        if (A_BF16) {
            scale = scale_from_amax(amax_from_words(aw));
            asm volatile("" : "+v"(scale));
        }
        const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)g.A, 0, M * K * (A_BF16 ? 2 : 1), 0x00020000);
        const int ct = tid - 512;
        const int arow = ct >> 3, ach = ct & 7;
        dg_v4i ra[NKS][A_LD];
#pragma unroll
        for (int j = 0; j < NKS; j++) {
            const int gk = j * 128 + ach * 16;
            const uint32_t vo = (arow < M && gk < K) ? ((uint32_t)arow * (uint32_t)K + (uint32_t)gk) * (A_BF16 ? 2u : 1u) : NC_DG_OOB;
#pragma unroll
            for (int h = 0; h < A_LD; h++) ra[j][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_a, vo, h * 16, 0);
        }
#pragma unroll
        for (int j = 0; j < NKS; j++) {
            dg_v4i v;
            if (A_BF16) {
                const uint32_t w[8] = {(uint32_t)ra[j][0][0], (uint32_t)ra[j][0][1], (uint32_t)ra[j][0][2], (uint32_t)ra[j][0][3],
                                       (uint32_t)ra[j][A_LD - 1][0], (uint32_t)ra[j][A_LD - 1][1], (uint32_t)ra[j][A_LD - 1][2],
                                       (uint32_t)ra[j][A_LD - 1][3]};
#pragma unroll
                for (int q = 0; q < 4; q++)
                    // no clamp needed: |x| <= amax gives |x*scale| <= 448*(1+2^-23), which rounds to 448 like the clamped value
                    v[q] = (int)e4m3_pack4_hw(bf16_lo(w[2 * q]) * scale, bf16_hi(w[2 * q]) * scale, bf16_lo(w[2 * q + 1]) * scale,
                                              bf16_hi(w[2 * q + 1]) * scale);
            } else {
                v = ra[j][0];
            }
            *(dg_v4i*)(&dgf_lds[j * 8192 + arow * 128 + ((ach ^ (arow & 7)) << 4)]) = v;      // (tiles past K hold zeros)
        }
        __syncthreads();                  // the panel is complete
        __syncthreads();                  // (the meeting of the K quarters)
        if (g.out_kind == 2 && g.out_amax) __syncthreads();
        return;
    }

    // ---- the multiplying waves: wave (cb, kq) asks for its weight rows at once and waits for the panel
    const int frow = lane & 15, kb = lane >> 4;
    const int cb = wave & 1, kq = wave >> 1;
    const int n0 = blockIdx.x * 32 + cb * 16;
    const int brow = n0 + frow;
    const int nq = (nksteps + 3) >> 2;                             // K-steps [kq * nq, (kq + 1) * nq) belong to quarter kq
    const int ks0 = kq * nq;
    const int nk = ks0 + nq <= nksteps ? nq : (nksteps > ks0 ? nksteps - ks0 : 0);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)g.B, 0, N * K, 0x00020000);
    dg_v4i rb[NKQ][2];
#pragma unroll
    for (int j = 0; j < NKQ; j++) {
        // (a lane's 32 K-bytes of a step are pieces kb and 4 + kb of its 128, on both sides: 64 contiguous bytes per row and instruction)
        const int gk = (ks0 + j) * 128 + kb * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t vo = (brow < N && j < nk && gk + h * 64 < K) ? (uint32_t)brow * (uint32_t)K + (uint32_t)gk : NC_DG_OOB;
            rb[j][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_b, vo, h * 64, 0);
        }
    }
    if (A_BF16) inv_a = 1.0f / scale_from_amax(amax_from_words(aw));
    __syncthreads();

    v4f acc[4];
#pragma unroll
    for (int i = 0; i < 4; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
    // no branch per K-step (the waits then count loads): a step past this quarter multiplies zero weight rows with some tile of the panel
#pragma unroll
    for (int j = 0; j < NKQ; j++) {
        const uint8_t* tile = dgf_lds + (j < nk ? ks0 + j : 0) * 8192;
        v8i bf;
        bf[0] = rb[j][0][0], bf[1] = rb[j][0][1], bf[2] = rb[j][0][2], bf[3] = rb[j][0][3];
        bf[4] = rb[j][1][0], bf[5] = rb[j][1][1], bf[6] = rb[j][1][2], bf[7] = rb[j][1][3];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int row = i * 16 + frow;
            const dg_v4i alo = *(const dg_v4i*)(tile + row * 128 + ((kb ^ (row & 7)) << 4));
            const dg_v4i ahi = *(const dg_v4i*)(tile + row * 128 + (((4 + kb) ^ (row & 7)) << 4));
            v8i af;
            af[0] = alo[0], af[1] = alo[1], af[2] = alo[2], af[3] = alo[3], af[4] = ahi[0], af[5] = ahi[1], af[6] = ahi[2], af[7] = ahi[3];
            acc[i] = MFMA_F8(acc[i], bf, af);
        }
    }

    // the later K quarters hand their sums to the first one (always added in the order 1, 2, 3)
    if (kq) {
        float* mp = meet + (((kq - 1) * 2 + cb) * 64 + lane) * 16;
#pragma unroll
        for (int i = 0; i < 4; i++) *(float4*)(mp + 4 * i) = make_float4(acc[i][0], acc[i][1], acc[i][2], acc[i][3]);
    }
    __syncthreads();
    float am = 0.f;
    if (!kq) {
#pragma unroll
        for (int q = 0; q < 3; q++) {
            const float* mp = meet + ((q * 2 + cb) * 64 + lane) * 16;
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float4 u = *(const float4*)(mp + 4 * i);
                acc[i][0] += u.x, acc[i][1] += u.y, acc[i][2] += u.z, acc[i][3] += u.w;
            }
        }
        // lane holds rows 16*i + frow, columns n0 + 4*kb .. +3
        const int n = n0 + 4 * kb;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = i * 16 + frow;
            if (m < M && n < N) {
                const float inv_b = dg_seg_scale(g, n);
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = (acc[i][r] * inv_a) * inv_b;
                if (g.out_kind == 1) {
                    float* o = (float*)g.out + (size_t)m * g.ldc + n;
                    for (int r = 0; r < 4 && n + r < N; r++) o[r] = g.softcap * tanhf(rbf(v[r]) / g.softcap);
                } else {
                    if (g.out_kind == 2) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const float t = relu_keep_nan(rbf(v[r]));
                            v[r] = rbf(t * t);
                            if (n + r < N) am = amax_join(am, v[r]);
                        }
                    }
                    bf16_t* o = (bf16_t*)g.out + (size_t)m * g.ldc + n;
                    if (n + 3 < N) *(uint2*)o = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
                    else
                        for (int r = 0; r < 4 && n + r < N; r++) o[r] = f32_to_bf16(v[r]);
                }
            }
        }
    }
    if (g.out_kind == 2 && g.out_amax) {
        am = wave_amax(am);
        if (!kq && lane == 0) red[cb] = am;
        __syncthreads();
        if (tid == 0) amax_publish(g.out_amax, amax_join(red[0], red[1]));
    }
}

// ------------------------------------------------------------------------------------------------
// Unsplit form for a wide output (lm_head): 17 .. 64 rows, K <= 2048, thousands of columns.  A workgroup of 8 waves converts the
// activation panel into LDS once and then owns 128 columns at a time (16 per wave, the whole of K, no meeting between waves), taking
// further blocks of 128 while there are any, so the panel is read and converted by at most as many workgroups as the chip has CUs
// instead of once per 64 columns.  Each wave asks for all weight rows of its block at once and multiplies K-step by K-step as they
// arrive.
template <bool A_BF16, int NKS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_decode_wide_kernel(DecodeGemmArgs g) {
    constexpr int A_LD = A_BF16 ? 2 : 1;
    extern __shared__ __align__(16) uint8_t dgw_lds[];            // NKS tiles of 8 KB
    __shared__ float red[8];

    NC_ARG_NOW(g.A); NC_ARG_NOW(g.a_amax); NC_ARG_NOW(g.inv_a); NC_ARG_NOW(g.B); NC_ARG_NOW(g.inv_b); NC_ARG_NOW(g.out); NC_ARG_NOW(g.out_kind);
    NC_ARG_NOW(g.out_amax); NC_ARG_NOW(g.ldc); NC_ARG_NOW(g.M); NC_ARG_NOW(g.N); NC_ARG_NOW(g.K);
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int frow = lane & 15, kb = lane >> 4;
    const int M = g.M, N = g.N, K = g.K;
    const int nblk = (N + 127) >> 7;

    AmaxWords aw = {};
    float inv_a = 0.f;
    if (A_BF16) aw = amax_load_scalar(g.a_amax);
    else inv_a = *g.inv_a;

    const __amdgpu_buffer_rsrc_t desc_a = __builtin_amdgcn_make_buffer_rsrc((void*)g.A, 0, M * K * (A_BF16 ? 2 : 1), 0x00020000);
    const __amdgpu_buffer_rsrc_t desc_b = __builtin_amdgcn_make_buffer_rsrc((void*)g.B, 0, N * K, 0x00020000);

    // activation panel: thread t converts chunk (row t >> 3, 16-byte piece t & 7) of every K-step tile
    const int arow = tid >> 3, ach = tid & 7;
    dg_v4i ra[NKS][A_LD], rb[NKS][2];
#pragma unroll
    for (int j = 0; j < NKS; j++) {
        const int gk = j * 128 + ach * 16;
        const uint32_t vo = (arow < M && gk < K) ? ((uint32_t)arow * (uint32_t)K + (uint32_t)gk) * (A_BF16 ? 2u : 1u) : NC_DG_OOB;
#pragma unroll
        for (int h = 0; h < A_LD; h++) ra[j][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_a, vo, h * 16, 0);
    }
    auto load_b = [&](int blk) {
        const int brow = blk * 128 + wave * 16 + frow;
#pragma unroll
        for (int j = 0; j < NKS; j++) {
            // (a lane's 32 K-bytes of a step are pieces kb and 4 + kb of its 128, on both sides: 64 contiguous bytes per row and instruction)
            const int gk = j * 128 + kb * 16;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const uint32_t vo = (brow < N && gk + h * 64 < K) ? (uint32_t)brow * (uint32_t)K + (uint32_t)gk : NC_DG_OOB;
                rb[j][h] = __builtin_amdgcn_raw_buffer_load_b128(desc_b, vo, h * 64, 0);
            }
        }
    };
    load_b(blockIdx.x);

    float scale = 1.f;
    if (A_BF16) {
        scale = scale_from_amax(amax_from_words(aw));
        inv_a = 1.0f / scale;
    }
#pragma unroll
    for (int j = 0; j < NKS; j++) {
        dg_v4i v;
        if (A_BF16) {
            const uint32_t w[8] = {(uint32_t)ra[j][0][0], (uint32_t)ra[j][0][1], (uint32_t)ra[j][0][2], (uint32_t)ra[j][0][3],
                                   (uint32_t)ra[j][A_LD - 1][0], (uint32_t)ra[j][A_LD - 1][1], (uint32_t)ra[j][A_LD - 1][2],
                                   (uint32_t)ra[j][A_LD - 1][3]};
#pragma unroll
            for (int q = 0; q < 4; q++)
                // no clamp needed: |x| <= amax gives |x*scale| <= 448*(1+2^-23), which rounds to 448 like the clamped value
                v[q] = (int)e4m3_pack4_hw(bf16_lo(w[2 * q]) * scale, bf16_hi(w[2 * q]) * scale, bf16_lo(w[2 * q + 1]) * scale,
                                          bf16_hi(w[2 * q + 1]) * scale);
        } else {
            v = ra[j][0];
        }
        *(dg_v4i*)(&dgw_lds[j * 8192 + arow * 128 + ((ach ^ (arow & 7)) << 4)]) = v;      // (tiles past K hold zeros)
    }
    __syncthreads();

    float am = 0.f;
    for (int blk = blockIdx.x; blk < nblk; blk += gridDim.x) {
        v4f acc[4];
#pragma unroll
        for (int i = 0; i < 4; i++) acc[i] = v4f{0.f, 0.f, 0.f, 0.f};
        // every tile of the panel, the ones past K included (zeros on both sides): no branch, so the waits count loads
#pragma unroll
        for (int j = 0; j < NKS; j++) {
            const uint8_t* tile = dgw_lds + j * 8192;
            v8i bf;
            bf[0] = rb[j][0][0], bf[1] = rb[j][0][1], bf[2] = rb[j][0][2], bf[3] = rb[j][0][3];
            bf[4] = rb[j][1][0], bf[5] = rb[j][1][1], bf[6] = rb[j][1][2], bf[7] = rb[j][1][3];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int row = i * 16 + frow;
                const dg_v4i alo = *(const dg_v4i*)(tile + row * 128 + ((kb ^ (row & 7)) << 4));
                const dg_v4i ahi = *(const dg_v4i*)(tile + row * 128 + (((4 + kb) ^ (row & 7)) << 4));
                v8i af;
                af[0] = alo[0], af[1] = alo[1], af[2] = alo[2], af[3] = alo[3], af[4] = ahi[0], af[5] = ahi[1], af[6] = ahi[2], af[7] = ahi[3];
                acc[i] = MFMA_F8(acc[i], bf, af);
            }
            __builtin_amdgcn_sched_barrier(0);          // (keeps the panel reads of later steps from being hoisted over this one)
        }
        // the next block's weight rows are on their way while this one's results leave
        if (blk + (int)gridDim.x < nblk) load_b(blk + gridDim.x);
        // lane holds rows 16*i + frow, columns n .. n + 3
        const int n = blk * 128 + wave * 16 + 4 * kb;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int m = i * 16 + frow;
            if (m < M && n < N) {
                const float inv_b = dg_seg_scale(g, n);
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = (acc[i][r] * inv_a) * inv_b;
                if (g.out_kind == 1) {
                    float* o = (float*)g.out + (size_t)m * g.ldc + n;
                    if (n + 3 < N && (g.ldc & 3) == 0 && ((uintptr_t)g.out & 15) == 0) {
                        float4 t;
                        t.x = g.softcap * tanhf(rbf(v[0]) / g.softcap), t.y = g.softcap * tanhf(rbf(v[1]) / g.softcap);
                        t.z = g.softcap * tanhf(rbf(v[2]) / g.softcap), t.w = g.softcap * tanhf(rbf(v[3]) / g.softcap);
                        *(float4*)o = t;
                    } else {
                        for (int r = 0; r < 4 && n + r < N; r++) o[r] = g.softcap * tanhf(rbf(v[r]) / g.softcap);
                    }
                } else {
                    if (g.out_kind == 2) {
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            const float t = relu_keep_nan(rbf(v[r]));
                            v[r] = rbf(t * t);
                            if (n + r < N) am = amax_join(am, v[r]);
                        }
                    }
                    bf16_t* o = (bf16_t*)g.out + (size_t)m * g.ldc + n;
                    if (n + 3 < N) *(uint2*)o = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
                    else
                        for (int r = 0; r < 4 && n + r < N; r++) o[r] = f32_to_bf16(v[r]);
                }
            }
        }
    }
    if (g.out_kind == 2 && g.out_amax) {
        am = wave_amax(am);
        if (lane == 0) red[wave] = am;
        __syncthreads();
        if (tid == 0) {
#pragma unroll
            for (int i = 1; i < 8; i++) am = amax_join(am, red[i]);
            amax_publish(g.out_amax, amax_join(am, red[0]));
        }
    }
}

namespace {
template <bool A_BF16, int NKS>
int launch_full(const DecodeGemmArgs& g, int nblk32, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    static bool reserved[64];
    constexpr int lds_bytes = NKS * 8192 + 6 * 4096;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev < 0 || dev >= 64 || !reserved[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)gemm_decode_full_kernel<A_BF16, NKS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm(decode): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
        if (dev >= 0 && dev < 64) reserved[dev] = true;
    }
    if (ev0) hipExtLaunchKernelGGL((gemm_decode_full_kernel<A_BF16, NKS>), dim3(nblk32), dim3(1024), lds_bytes, s, ev0, ev1, 0, g);
    else hipLaunchKernelGGL((gemm_decode_full_kernel<A_BF16, NKS>), dim3(nblk32), dim3(1024), lds_bytes, s, g);
    return 0;
}
}  // namespace

namespace {
template <bool A_BF16, int NKS>
int launch_wide(const DecodeGemmArgs& g, int grid, hipStream_t s, hipEvent_t ev0, hipEvent_t ev1) {
    static bool reserved[64];
    constexpr int lds_bytes = NKS * 8192;
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev < 0 || dev >= 64 || !reserved[dev]) {
        const hipError_t e = hipFuncSetAttribute((const void*)gemm_decode_wide_kernel<A_BF16, NKS>, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
        if (e != hipSuccess) NC_FAIL(-2, "fp8_gemm(decode): cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
        if (dev >= 0 && dev < 64) reserved[dev] = true;
    }
    if (ev0) hipExtLaunchKernelGGL((gemm_decode_wide_kernel<A_BF16, NKS>), dim3(grid), dim3(512), lds_bytes, s, ev0, ev1, 0, g);
    else hipLaunchKernelGGL((gemm_decode_wide_kernel<A_BF16, NKS>), dim3(grid), dim3(512), lds_bytes, s, g);
    return 0;
}
}  // namespace

// Whether a single-split launch runs the wide form: at least one block of 128 columns per CU.
static bool dg_wide_form(int M, int N, int K, bool made) {
    return !made && M > 16 && M <= 64 && K <= NC_DGF_MAX_K && (N + 127) / 128 >= 256 && (int64_t)N * K < ((int64_t)1 << 31);
}

// Whether nc_launch_gemm_decode, left to choose (ksplits 0), runs the unsplit form: enough 32-column blocks to occupy half the chip
// and few enough to run in one round.
static bool dg_full_form(int M, int N, int K, bool made, int out_kind) {
    const int nblk32 = (N + 31) / 32;
    return out_kind == 2 && !made && M > 16 && M <= 64 && K <= NC_DGF_MAX_K && nblk32 >= 128 && nblk32 <= 256 && (int64_t)N * K < ((int64_t)1 << 31);
}

// ------------------------------------------------------------------------------------------------
// out = epilogue((sum over splits of partials) * inv_a * inv_w[segment]) -- the finishing pass for callers that
// need the linear's output materialised (the MLP activation, and the stand-alone API).
__global__ __launch_bounds__(256) void finish_partials_kernel(const float* __restrict__ parts, int nsplit, size_t split_stride,
                                                              const uint32_t* __restrict__ a_amax, const float* __restrict__ inv_a_ptr,
                                                              const float* __restrict__ inv_b,
                                                              NcGemmSegs segs, void* __restrict__ out, int out_kind, float softcap,
                                                              uint32_t* __restrict__ out_amax, int M, int N, int ldc) {
    NC_ARG_NOW(parts); NC_ARG_NOW(nsplit); NC_ARG_NOW(split_stride); NC_ARG_NOW(a_amax); NC_ARG_NOW(inv_a_ptr); NC_ARG_NOW(inv_b);
    NC_ARG_NOW(out); NC_ARG_NOW(out_kind); NC_ARG_NOW(out_amax); NC_ARG_NOW(M); NC_ARG_NOW(N); NC_ARG_NOW(ldc);
    __shared__ float red[4];
    // asked for now, looked at after the first batch of partial sums has been requested
    const uint32_t amax_lane = a_amax ? amax_load_lane(a_amax) : 0u;
    float inv_a = a_amax ? 0.f : *inv_a_ptr;
    bool have_inv_a = a_amax == nullptr;
    const int n4 = N / 4;
    float am = 0.f;
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < (size_t)M * n4; i += (size_t)gridDim.x * 256) {
        const int m = (int)(i / n4), n = (int)(i % n4) * 4;
        float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
        // the weight scale of the column's segment is asked for together with the partial sums, not after them
        int sg = 0;
#pragma unroll
        for (int k = 0; k < 3; k++)
            if (k + 1 < segs.nseg && n >= segs.end[k]) sg = k + 1;
        const float ib = inv_b[sg];
        // eight splits at a time: loads first, sums after in split order (one round trip to memory, not one per split)
        const float* pp = parts + (size_t)m * N + n;
        for (int s0 = 0; s0 < nsplit; s0 += 8) {
            float4 p[8];
#pragma unroll
            for (int u = 0; u < 8; u++) p[u] = *(const float4*)(pp + (size_t)(s0 + u < nsplit ? s0 + u : s0) * split_stride);
            if (!have_inv_a) inv_a = 1.0f / scale_from_amax(amax_from_lanes(amax_lane)), have_inv_a = true;
#pragma unroll
            for (int u = 0; u < 8; u++)
                if (s0 + u < nsplit) a.x += p[u].x, a.y += p[u].y, a.z += p[u].z, a.w += p[u].w;
        }
        float v[4] = {(a.x * inv_a) * ib, (a.y * inv_a) * ib, (a.z * inv_a) * ib, (a.w * inv_a) * ib};
        if (out_kind == 1) {
            float* o = (float*)out + (size_t)m * ldc + n;
#pragma unroll
            for (int r = 0; r < 4; r++) o[r] = softcap * tanhf(rbf(v[r]) / softcap);
        } else {
            if (out_kind == 2) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const float t = relu_keep_nan(rbf(v[r]));
                    v[r] = rbf(t * t);
                    am = amax_join(am, v[r]);
                }
            }
            *(uint2*)((bf16_t*)out + (size_t)m * ldc + n) = make_uint2(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]));
        }
    }
    if (out_kind == 2 && out_amax) {
        am = wave_amax(am);
        if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = am;
        __syncthreads();
        if (threadIdx.x == 0) {
            am = amax_join(amax_join(red[0], red[1]), amax_join(red[2], red[3]));
            amax_publish(out_amax, am);
        }
    }
}

int nc_launch_finish_partials(const float* parts, int nsplit, const uint32_t* a_amax, const float* inv_a, const float* inv_b,
                              NcGemmSegs segs, void* out, int out_kind, float softcap, uint32_t* out_amax, int M, int N, int ldc,
                              hipStream_t s) {
    NC_CHECK_ARG(parts && (a_amax || inv_a) && inv_b && out && nsplit >= 1 && N % 4 == 0, "finish_partials: bad arguments");
    NC_CHECK_ARG(ldc >= N && out_kind >= 0 && out_kind <= 2, "finish_partials: bad output description");
    if (out_kind != 1) NC_CHECK_ARG(((uintptr_t)out & 7) == 0 && ldc % 4 == 0, "finish_partials: bf16 output needs 8-byte alignment and ldc %% 4 == 0");
    NcProfScope prof(3, 4.0 * nsplit * M * N, s);
    int grid = (int)(((size_t)M * (N / 4) + 255) / 256);
    if (grid > 2048) grid = 2048;
    hipLaunchKernelGGL(finish_partials_kernel, dim3(grid), dim3(256), 0, s, parts, nsplit, (size_t)M * N, a_amax, inv_a, inv_b, segs,
                       out, out_kind, softcap, out_amax, M, N, ldc);
    NC_CHECK_LAUNCH("finish_partials");
    return 0;
}

// How many K splits a [M<=128] x [N,K] linear is cut into.  Measured on d26 shapes at M=64: a workgroup that
// covers one 512-wide K chunk (a single round of loads) finishes in ~6 us and every further chunk it walks adds
// ~3 us of exposed latency, so K is split over workgroups.  Only a layer with hundreds of column blocks of its own
// (lm_head) runs unsplit with the epilogue in the GEMM.
int nc_gemm_decode_splits(int N, int K) {
    const int nblk = (N + 63) / 64;
    const int nksteps = (K + 127) / 128;
    if (N % 4 != 0 || nblk >= 256) return 1;
    // as many splits as keep the launch within one round of the 256 CUs (a second round of workgroups costs more than longer
    // K runs), and at most 8: beyond that the consumer pays more for the partial sums it has to read than the GEMM gains
    int ks = 256 / nblk;
    if (ks > 8) ks = 8;
    if (ks < 1) ks = 1;
    // a short K (at most 16 steps) is cut in four at most: each workgroup still makes one trip (four steps), and the consumer reads
    // four partial sums per output instead of seven (measured equal to slightly faster, and 1.3 MB less to write and read back)
    if (nksteps <= 16 && ks > 4) ks = 4;
    const int kps = (nksteps + ks - 1) / ks;
    return (nksteps + kps - 1) / kps;
}

// room for the partial sums of the split count nc_gemm_decode_splits() picks (what a forward pass needs)
size_t nc_gemm_decode_partial_bytes_auto(int M, int N, int K) {
    const int ks = nc_gemm_decode_splits(N, K);
    return ks > 1 ? (size_t)ks * M * N * sizeof(float) : 0;
}

// room for the partial sums of any split count a caller may ask for (at most 16, and no more than there are K-steps)
size_t nc_gemm_decode_partial_bytes(int M, int N, int K) {
    if (N % 4 != 0) return 0;
    const int nksteps = (K + 127) / 128;
    const int ks = nksteps < 16 ? nksteps : 16;
    return ks > 1 ? (size_t)ks * M * N * sizeof(float) : 0;
}

// ksplits: 0 = nc_gemm_decode_splits().  With more than one split the result is left in `partials`
// ([ksplits][M][N] fp32, raw sums) and *ksplits_out says how many; out/out_kind are then unused.
int nc_launch_gemm_decode(const void* a, int a_is_bf16, const uint32_t* a_amax, const float* inv_a, const uint8_t* b,
                          const float* inv_b, NcGemmSegs segs, void* out, int out_kind, float softcap, uint32_t* out_amax, int M,
                          int N, int K, int ldc, float* partials, size_t partial_bytes, int ksplits, int* ksplits_out, hipStream_t s,
                          const NcRowRecipe* recipe) {
    const bool made = recipe && recipe->kind != 0;
    NC_CHECK_ARG((a || made) && b, "fp8_gemm(decode): null pointer");
    NC_CHECK_ARG(made || (a_is_bf16 ? (a_amax != nullptr) : (inv_a != nullptr)), "fp8_gemm(decode): activation scale missing");
    if (made) {
        NC_CHECK_ARG(M <= NC_RECIPE_MAX_ROWS && K % 8 == 0 && K <= (recipe->kind == 1 ? 2048 : NC_RECIPE_MAX_K) && recipe->amax_out,
                     "fp8_gemm(decode): a row recipe takes at most %d rows of at most %d elements", NC_RECIPE_MAX_ROWS, NC_RECIPE_MAX_K);
        NC_CHECK_ARG(recipe->kind == 1 ? (recipe->x_in && recipe->x_out && recipe->x_in != recipe->x_out && (!recipe->resid_lambda || (recipe->x0 && recipe->x0_lambda)))
                                       : (recipe->kind == 2 && recipe->padd.parts), "fp8_gemm(decode): incomplete row recipe");
        NC_CHECK_ARG(!recipe->padd.parts || (recipe->padd.nsplit >= 1 && recipe->padd.a_amax && recipe->padd.inv_b && recipe->padd.ld >= K),
                     "fp8_gemm(decode): bad partial-sum source in the row recipe");
    }
    NC_CHECK_ARG(M >= 1 && M <= 128 && N > 0 && K > 0, "fp8_gemm(decode): bad shape M=%d N=%d K=%d (M <= 128)", M, N, K);
    NC_CHECK_ARG(K % 16 == 0, "fp8_gemm: K=%d must be a multiple of 16", K);
    NC_CHECK_ARG(((uintptr_t)a & 15) == 0 && ((uintptr_t)b & 15) == 0, "fp8_gemm: operands must be 16-byte aligned");
    const int nksteps = (K + 127) / 128;
    const bool full = ksplits <= 0 && dg_full_form(M, N, K, made, out_kind);
    if (full) ksplits = 1;
    if (ksplits <= 0) ksplits = nc_gemm_decode_splits(N, K);
    NC_CHECK_ARG(ksplits <= 16, "fp8_gemm(decode): at most 16 K splits, got %d", ksplits);
    if (ksplits > nksteps) ksplits = nksteps;
    int kps = (nksteps + ksplits - 1) / ksplits;
    ksplits = (nksteps + kps - 1) / kps;
    if (ksplits > 1) {
        NC_CHECK_ARG(N % 4 == 0, "fp8_gemm(decode): split-K needs N %% 4 == 0");
        NC_CHECK_ARG(partials && partial_bytes >= (size_t)ksplits * M * N * sizeof(float) && ((uintptr_t)partials & 15) == 0,
                     "fp8_gemm(decode): %d splits need %zu bytes of 16-byte aligned partial-sum workspace", ksplits,
                     (size_t)ksplits * M * N * sizeof(float));
    } else {
        NC_CHECK_ARG(out && inv_b, "fp8_gemm(decode): null output");
        NC_CHECK_ARG(ldc >= N, "fp8_gemm: ldc=%d < N=%d", ldc, N);
        NC_CHECK_ARG(out_kind >= 0 && out_kind <= 2, "fp8_gemm: out_kind must be 0, 1 or 2");
        NC_CHECK_ARG(segs.nseg >= 1 && segs.nseg <= 4 && segs.end[segs.nseg - 1] == N, "fp8_gemm: bad column segments");
        for (int i = 0; i + 1 < segs.nseg; i++)
            NC_CHECK_ARG(segs.end[i] % 4 == 0 && segs.end[i] < segs.end[i + 1], "fp8_gemm: segment ends must be increasing multiples of 4");
        if (out_kind != 1) NC_CHECK_ARG(((uintptr_t)out & 7) == 0 && ldc % 4 == 0, "fp8_gemm: bf16 output needs 8-byte alignment and ldc %% 4 == 0");
    }
    if (ksplits_out) *ksplits_out = ksplits;

    const int nblk = (N + 63) / 64;
    DecodeGemmArgs g;
    g.A = a, g.a_amax = a_amax, g.inv_a = inv_a, g.B = b, g.inv_b = inv_b, g.segs = segs, g.out = out, g.out_kind = out_kind;
    g.softcap = softcap, g.ldc = ldc, g.out_amax = out_amax, g.partial_out = partials;
    g.ksplits = ksplits, g.ksteps_per_split = kps, g.M = M, g.N = N, g.K = K;
    g.recipe = made ? *recipe : NcRowRecipe{};
    // rows of the MFMA block: the A panel in LDS (and its staging, zero rows included) is sized by it, so a small batch takes a small
    // block (batch 8: 1.50 -> 1.35 ms per d26 step with 16 rows instead of 64)
    const int MB = (made || M <= 16) ? 1 : (M <= 32 ? 2 : (M <= 48 ? 3 : (M <= 64 ? 4 : 8)));
    const bool wide = ksplits == 1 && !full && dg_wide_form(M, N, K, made);
    const bool onetrip = kps <= 8 && (int64_t)N * K < ((int64_t)1 << 31);
    // the one-trip, unsplit and wide forms hand their event pair to the launch itself when the profiler is on (the kernel's own begin and end,
    // no marker packets around it); the chunk-walking kernel keeps the bracketing pair
    const bool own_events = wide || full || onetrip;
    hipEvent_t ev0 = nullptr, ev1 = nullptr;
    if (own_events && !nc_prof_take(1, 2.0 * M * N * K, ((int64_t)N << 32) | (uint32_t)K, &ev0, &ev1)) ev0 = ev1 = nullptr;
    NcProfScope prof(own_events ? -1 : 1, 2.0 * M * N * K, s, ((int64_t)N << 32) | (uint32_t)K);
    if (wide) {
        const int nblk128 = (N + 127) / 128, cus = nc_cu_count();
        const int grid = nblk128 < cus ? nblk128 : cus;
        int rc;
        if (nksteps <= 10) rc = a_is_bf16 ? launch_wide<true, 10>(g, grid, s, ev0, ev1) : launch_wide<false, 10>(g, grid, s, ev0, ev1);
        else if (nksteps <= 13) rc = a_is_bf16 ? launch_wide<true, 13>(g, grid, s, ev0, ev1) : launch_wide<false, 13>(g, grid, s, ev0, ev1);
        else rc = a_is_bf16 ? launch_wide<true, 16>(g, grid, s, ev0, ev1) : launch_wide<false, 16>(g, grid, s, ev0, ev1);
        if (rc) return rc;
        NC_CHECK_LAUNCH("fp8_gemm(decode)");
        return 0;
    }
    if (full) {
        const int nblk32 = (N + 31) / 32;
        int rc;
        if (nksteps <= 10) rc = a_is_bf16 ? launch_full<true, 10>(g, nblk32, s, ev0, ev1) : launch_full<false, 10>(g, nblk32, s, ev0, ev1);
        else if (nksteps <= 13) rc = a_is_bf16 ? launch_full<true, 13>(g, nblk32, s, ev0, ev1) : launch_full<false, 13>(g, nblk32, s, ev0, ev1);
        else rc = a_is_bf16 ? launch_full<true, 16>(g, nblk32, s, ev0, ev1) : launch_full<false, 16>(g, nblk32, s, ev0, ev1);
        if (rc) return rc;
        NC_CHECK_LAUNCH("fp8_gemm(decode)");
        return 0;
    }
    dim3 grid(nblk, ksplits), block(256);
#define OT_LAUNCH_N(MB_, MODE_, NSET_, WR_)                                                                                    \
    do {                                                                                                                       \
        constexpr int lds_bytes__ = NSET_ * MB_ * 16 * WR_ * 512;                                                              \
        if (lds_bytes__ > 65536) {                                                                                             \
            static bool reserved__[64];                                                                                        \
            int dev__ = 0;                                                                                                     \
            (void)hipGetDevice(&dev__);                                                                                        \
            if (dev__ < 0 || dev__ >= 64 || !reserved__[dev__]) {                                                              \
                const hipError_t e__ = hipFuncSetAttribute((const void*)gemm_decode_onetrip_kernel<MB_, MODE_, NSET_, WR_>,    \
                                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes__);           \
                if (e__ != hipSuccess) NC_FAIL(-2, "fp8_gemm(decode): cannot reserve %d bytes of LDS: %s", lds_bytes__, hipGetErrorString(e__)); \
                if (dev__ >= 0 && dev__ < 64) reserved__[dev__] = true;                                                        \
            }                                                                                                                  \
        }                                                                                                                      \
        if (ev0)                                                                                                               \
            hipExtLaunchKernelGGL((gemm_decode_onetrip_kernel<MB_, MODE_, NSET_, WR_>), grid, dim3(256 * WR_), lds_bytes__, s, ev0, ev1, 0, g); \
        else                                                                                                                   \
            hipLaunchKernelGGL((gemm_decode_onetrip_kernel<MB_, MODE_, NSET_, WR_>), grid, dim3(256 * WR_), lds_bytes__, s, g); \
    } while (0)
#define OT_LAUNCH(MB_, MODE_)                       \
    do {                                            \
        if (kps <= 4) OT_LAUNCH_N(MB_, MODE_, 1, 1); \
        else OT_LAUNCH_N(MB_, MODE_, 2, 1);         \
    } while (0)
    if (onetrip) {
        if (made) {
            if (recipe->kind == 1) OT_LAUNCH(1, 2);
            else OT_LAUNCH(1, 3);
        } else if (MB == 1) {
            if (a_is_bf16) OT_LAUNCH(1, 1);
            else OT_LAUNCH(1, 0);
        } else if (MB == 2) {
            if (a_is_bf16) OT_LAUNCH(2, 1);
            else OT_LAUNCH(2, 0);
        } else if (MB == 3) {
            if (a_is_bf16) OT_LAUNCH(3, 1);
            else OT_LAUNCH(3, 0);
        } else if (MB == 4) {
            if (a_is_bf16) OT_LAUNCH(4, 1);
            else OT_LAUNCH(4, 0);
        } else {
            // 65 .. 128 rows: eight waves, two row halves of 64
            if (kps <= 4) {
                if (a_is_bf16) OT_LAUNCH_N(4, 1, 1, 2);
                else OT_LAUNCH_N(4, 0, 1, 2);
            } else {
                if (a_is_bf16) OT_LAUNCH_N(4, 1, 2, 2);
                else OT_LAUNCH_N(4, 0, 2, 2);
            }
        }
    } else if (MB == 1) {
        if (made && recipe->kind == 1) hipLaunchKernelGGL((gemm_decode_kernel<1, 2>), grid, block, 0, s, g);
        else if (made) hipLaunchKernelGGL((gemm_decode_kernel<1, 3>), grid, block, 0, s, g);
        else if (a_is_bf16) hipLaunchKernelGGL((gemm_decode_kernel<1, 1>), grid, block, 0, s, g);
        else hipLaunchKernelGGL((gemm_decode_kernel<1, 0>), grid, block, 0, s, g);
    } else if (MB == 2) {
        if (a_is_bf16) hipLaunchKernelGGL((gemm_decode_kernel<2, 1>), grid, block, 0, s, g);
        else hipLaunchKernelGGL((gemm_decode_kernel<2, 0>), grid, block, 0, s, g);
    } else if (MB == 3) {
        if (a_is_bf16) hipLaunchKernelGGL((gemm_decode_kernel<3, 1>), grid, block, 0, s, g);
        else hipLaunchKernelGGL((gemm_decode_kernel<3, 0>), grid, block, 0, s, g);
    } else if (MB == 4) {
        if (a_is_bf16) hipLaunchKernelGGL((gemm_decode_kernel<4, 1>), grid, block, 0, s, g);
        else hipLaunchKernelGGL((gemm_decode_kernel<4, 0>), grid, block, 0, s, g);
    } else {
        if (a_is_bf16) hipLaunchKernelGGL((gemm_decode_kernel<8, 1>), grid, block, 0, s, g);
        else hipLaunchKernelGGL((gemm_decode_kernel<8, 0>), grid, block, 0, s, g);
    }
    NC_CHECK_LAUNCH("fp8_gemm(decode)");
    return 0;
}
