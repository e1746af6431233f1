// Row kernels of the decode step: embedding + norm + smear, residual mix + RMSNorm, relu^2, and the
// fused rotary / QK-norm / value-embedding gate / KV-cache append.
//
// The reference runs these as separate eager bf16 ops (nanochat/gpt.py:42-43, 57-65, 94-104, 471-508),
// each of which rounds its result to bf16.  The kernels keep values in fp32 registers but apply rbf()
// (round to bf16) at every point where the eager graph materialises a bf16 tensor, so results agree
// with the eager sequence instead of with an idealised fused formula.
//
// All of them are HBM/L2-bandwidth bound with tiny footprints at decode (a few hundred KB); the point
// of fusing is launch count, and producing the amax of the normalised row for the FP8 quantizer that
// follows (atomicMax on the fp32 bit pattern, valid because the values are non-negative).
#include "nc_common.h"
#include "nc_kernels.h"
#include "nc_rope.h"

__device__ __forceinline__ void block_amax_commit(float local_abs_max, uint32_t* amax_ws, float* red) {
    if (!amax_ws) return;
    float m = wave_amax(local_abs_max);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6, nw = blockDim.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = m;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int i = 1; i < nw; i++) m = amax_join(m, red[i]);
        amax_publish(amax_ws, m);
    }
}

// ------------------------------------------------------------------------------------------------
// x_out[b,t] = smear(norm(wte[idx[b,t]])), prev_out[b] = norm(wte[idx[b,T-1]])      (gpt.py:471-492)
// One block of 256 threads per token.  Row buffers live in LDS (fp32), cols <= 8192.
__global__ __launch_bounds__(256) void embed_norm_smear_kernel(const int64_t* __restrict__ idx, const bf16_t* __restrict__ wte,
                                                               const float* __restrict__ smear_w, const float* __restrict__ smear_lambda,
                                                               const bf16_t* __restrict__ prev_in, bf16_t* __restrict__ prev_out,
                                                               bf16_t* __restrict__ x_out, bf16_t* __restrict__ x0_out, int T, int E,
                                                               int vocab_rows, uint32_t* __restrict__ clear_words, int n_clear) {
    extern __shared__ float rowbuf[];          // [2][E]: this token, previous token (both normalised, bf16 values)
    __shared__ float red[8];
    // first kernel of a forward pass: it also zeroes the pass's amax slots and arrival counters
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n_clear; i += gridDim.x * 256) clear_words[i] = 0u;
    const int row = blockIdx.x, b = row / T, t = row % T;
    const bool use_prev_token = (T > 1 && t >= 1);
    const bool use_prev_cache = (T == 1 && prev_in != nullptr);

    for (int which = 0; which < (use_prev_token ? 2 : 1); which++) {
        int64_t tok = idx[(size_t)b * T + t - which];
        // An id outside the table never reads out of bounds; its row becomes NaN, which the tensorwise scales carry into every
        // logit of the call: the reference's nn.Embedding raises for such an id (gpt.py:470), a kernel cannot, and a silently
        // substituted row would be worse.  (The host refuses such ids in prompts and forced tokens before they get here.)
        const bool bad_id = tok < 0 || tok >= vocab_rows;
        if (bad_id) tok = 0;
        const bf16_t* e = wte + (size_t)tok * E;
        float ss = 0.f;
        for (int c = threadIdx.x; c < E; c += 256) {
            float v = bad_id ? __uint_as_float(0x7fc00000u) : bf16_to_f32(e[c]);
            rowbuf[which * E + c] = v;
            ss += v * v;
        }
        ss = block_sum<4>(ss, red);
        const float rstd = 1.0f / sqrtf(ss / (float)E + RMS_EPS);
        for (int c = threadIdx.x; c < E; c += 256) rowbuf[which * E + c] = rbf(rowbuf[which * E + c] * rstd);
        __syncthreads();
    }
    if (t == T - 1)
        for (int c = threadIdx.x; c < E; c += 256) prev_out[(size_t)b * E + c] = f32_to_bf16(rowbuf[c]);

    float gate = 0.f;
    if (use_prev_token || use_prev_cache) {
        // gate = bf16(lambda) * sigmoid(W_s . x[:24]); every product of the chain is a bf16 tensor in eager mode
        float dot = 0.f;
        for (int c = 0; c < 24; c++) dot += rowbuf[c] * rbf(smear_w[c]);
        gate = rbf(rbf(*smear_lambda) * rbf(sigmoidf_(rbf(dot))));
    }
    for (int c = threadIdx.x; c < E; c += 256) {
        float v = rowbuf[c];
        if (use_prev_token) v = rbf(v + rbf(gate * rowbuf[E + c]));
        else if (use_prev_cache) v = rbf(v + rbf(gate * bf16_to_f32(prev_in[(size_t)b * E + c])));
        x_out[(size_t)row * E + c] = f32_to_bf16(v);
        if (x0_out) x0_out[(size_t)row * E + c] = f32_to_bf16(v);      // the copy the per-layer residual mix reads (gpt.py:495)
    }
}

// The same for one token per row (decode) with E % 8 == 0 and E <= 2048: thread c owns eight consecutive channels, the row and the
// previous token's row are one 16-byte load each, asked for together with the gate weights, and the normalised row stays in
// registers except for the 24 channels the gate reads.
__global__ __launch_bounds__(256) void embed_norm_smear_decode_kernel(const int64_t* __restrict__ idx, const bf16_t* __restrict__ wte,
                                                                      const float* __restrict__ smear_w,
                                                                      const float* __restrict__ smear_lambda,
                                                                      const bf16_t* __restrict__ prev_in, bf16_t* __restrict__ prev_out,
                                                                      bf16_t* __restrict__ x_out, bf16_t* __restrict__ x0_out, int E,
                                                                      int vocab_rows, uint32_t* __restrict__ clear_words, int n_clear) {
    __shared__ float red[8];
    __shared__ float head[24];
    const int b = blockIdx.x, c0 = threadIdx.x * 8;
    const bool mine = c0 < E;
    int64_t tok = idx[b];
    const bool bad_id = tok < 0 || tok >= vocab_rows;      // never read out of bounds: the row becomes NaN (see the kernel above)
    if (bad_id) tok = 0;
    uint4 ev = make_uint4(0, 0, 0, 0), pv = make_uint4(0, 0, 0, 0);
    if (mine) {
        ev = *(const uint4*)(wte + (size_t)tok * E + c0);
        if (prev_in) pv = *(const uint4*)(prev_in + (size_t)b * E + c0);
    }
    const float sw = (threadIdx.x & 63) < 24 ? smear_w[threadIdx.x & 63] : 0.f;      // lane c of every wave holds gate weight c
    const float lam = *smear_lambda;
    // first kernel of a forward pass: it also zeroes the pass's amax slots and arrival counters
    for (int i = blockIdx.x * 256 + threadIdx.x; i < n_clear; i += gridDim.x * 256) clear_words[i] = 0u;

    const uint32_t ew[4] = {ev.x, ev.y, ev.z, ev.w};
    float v[8], ss = 0.f;
#pragma unroll
    for (int j = 0; j < 4; j++) v[2 * j] = bf16_lo(ew[j]), v[2 * j + 1] = bf16_hi(ew[j]);
    if (bad_id) {
#pragma unroll
        for (int j = 0; j < 8; j++) v[j] = __uint_as_float(0x7fc00000u);
    }
#pragma unroll
    for (int j = 0; j < 8; j++) ss += v[j] * v[j];
    ss = block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)E + RMS_EPS);
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = rbf(v[j] * rstd);
    if (mine) *(uint4*)(prev_out + (size_t)b * E + c0) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
    if (prev_in) {
        if (threadIdx.x < 3) {
#pragma unroll
            for (int j = 0; j < 8; j++) head[c0 + j] = v[j];
        }
        __syncthreads();
        // gate = bf16(lambda) * sigmoid(W_s . x[:24]); every product of the chain is a bf16 tensor in eager mode
        float dot = 0.f;
        for (int c = 0; c < 24; c++) dot += head[c] * rbf(__shfl(sw, c));
        const float gate = rbf(rbf(lam) * rbf(sigmoidf_(rbf(dot))));
        const uint32_t pw[4] = {pv.x, pv.y, pv.z, pv.w};
#pragma unroll
        for (int j = 0; j < 4; j++) {
            v[2 * j] = rbf(v[2 * j] + rbf(gate * bf16_lo(pw[j])));
            v[2 * j + 1] = rbf(v[2 * j + 1] + rbf(gate * bf16_hi(pw[j])));
        }
    }
    if (mine) {
        const uint4 o = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
        *(uint4*)(x_out + (size_t)b * E + c0) = o;
        if (x0_out) *(uint4*)(x0_out + (size_t)b * E + c0) = o;      // the copy the per-layer residual mix reads (gpt.py:495)
    }
}

// ------------------------------------------------------------------------------------------------
// x1 = x (+ add);  [backout_save = x1];  x2 = rl*x1 + xl*x0  |  x1 - bl*backout_src  |  x1;
// x = x2;  xn = rms_norm(x2);  amax(xn).                                    (gpt.py:500, 151-152, 503-508)
__global__ __launch_bounds__(256) void mix_norm_kernel(bf16_t* __restrict__ x, const bf16_t* __restrict__ add, const bf16_t* __restrict__ x0,
                                                       const float* __restrict__ resid_lambda, const float* __restrict__ x0_lambda,
                                                       const float* __restrict__ backout_lambda, const bf16_t* __restrict__ backout_src,
                                                       bf16_t* __restrict__ backout_save, bf16_t* __restrict__ xn_out, int cols,
                                                       uint32_t* __restrict__ amax_ws) {
    extern __shared__ float rowbuf[];
    __shared__ float red[8];
    const size_t base = (size_t)blockIdx.x * cols;
    const float rl = resid_lambda ? rbf(*resid_lambda) : 0.f;
    const float xl = x0_lambda ? rbf(*x0_lambda) : 0.f;
    const float bl = backout_lambda ? rbf(*backout_lambda) : 0.f;
    float ss = 0.f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        float v = bf16_to_f32(x[base + c]);
        if (add) v = rbf(v + bf16_to_f32(add[base + c]));
        if (backout_save) backout_save[base + c] = f32_to_bf16(v);
        if (resid_lambda) v = rbf(rbf(rl * v) + rbf(xl * bf16_to_f32(x0[base + c])));
        else if (backout_lambda) v = rbf(v - rbf(bl * bf16_to_f32(backout_src[base + c])));
        if (add || resid_lambda || backout_lambda) x[base + c] = f32_to_bf16(v);
        rowbuf[c] = v;
        ss += v * v;
    }
    ss = block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)cols + RMS_EPS);
    float am = 0.f;
    for (int c = threadIdx.x; c < cols; c += 256) {
        const bf16_t o = f32_to_bf16(rowbuf[c] * rstd);
        xn_out[base + c] = o;
        am = amax_fold(am, bf16_to_f32(o));
    }
    block_amax_commit(am, amax_ws, red);
}

// Same contract as mix_norm_kernel for cols % 8 == 0 and cols <= 2048 * NV: the row stays in registers,
// eight bf16 per 16-byte access, one reduction, one pass over memory.
// PARTS: the addend arrives as split partial sums (decode).  Without them the kernel needs a third of the registers, and the
// thousands of one-row workgroups of a prefill fit the chip in one round instead of two.
template <int NV, bool PARTS>
__global__ __launch_bounds__(256) void mix_norm_vec_kernel(bf16_t* __restrict__ x, const bf16_t* __restrict__ add, NcPartialSrc padd,
                                                           const bf16_t* __restrict__ x0, const float* __restrict__ resid_lambda,
                                                           const float* __restrict__ x0_lambda, const float* __restrict__ backout_lambda,
                                                           const bf16_t* __restrict__ backout_src, bf16_t* __restrict__ backout_save,
                                                           bf16_t* __restrict__ xn_out, int cols, uint32_t* __restrict__ amax_ws,
                                                           int32_t* __restrict__ bump, int bump_by) {
    NC_ARG_NOW(x); NC_ARG_NOW(add); NC_ARG_NOW(padd.parts); NC_ARG_NOW(padd.nsplit); NC_ARG_NOW(padd.ld); NC_ARG_NOW(padd.split_stride);
    NC_ARG_NOW(padd.a_amax); NC_ARG_NOW(padd.inv_b); NC_ARG_NOW(x0); NC_ARG_NOW(resid_lambda); NC_ARG_NOW(x0_lambda);
    NC_ARG_NOW(backout_lambda); NC_ARG_NOW(backout_src); NC_ARG_NOW(backout_save); NC_ARG_NOW(xn_out); NC_ARG_NOW(cols); NC_ARG_NOW(amax_ws);
    __shared__ float red[8];
    const size_t base = (size_t)blockIdx.x * cols;
    const bool has_parts = PARTS && padd.parts != nullptr;
    const bool writes_x = add || has_parts || resid_lambda || backout_lambda;
    const bf16_t* zsrc = resid_lambda ? x0 : (backout_lambda ? backout_src : nullptr);

    // ---- every load the row needs is issued before anything waits for one: the kernel then costs one trip to memory, not one
    // per operand (the operands are a few KB, so the trips, not the bytes, are its whole duration)
    const float rl_raw = resid_lambda ? *resid_lambda : 0.f;
    const float xl_raw = x0_lambda ? *x0_lambda : 0.f;
    const float bl_raw = backout_lambda ? *backout_lambda : 0.f;
    const float p_inv_b = has_parts ? padd.inv_b[0] : 0.f;
    const uint32_t p_amax_lane = has_parts ? amax_load_lane(padd.a_amax) : 0u;
    uint4 xv[NV], av[NV], zv[NV];
    float4 a0[PARTS ? NV : 1][8], a1[PARTS ? NV : 1][8];
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int c = (threadIdx.x + it * 256) * 8;
        if (c < cols) {
            xv[it] = *(const uint4*)(x + base + c);
            if (add) av[it] = *(const uint4*)(add + base + c);
            if (zsrc) zv[it] = *(const uint4*)(zsrc + base + c);
            if (has_parts) {
                const float* pp = padd.parts + (size_t)blockIdx.x * padd.ld + c;
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    const float* q = pp + (size_t)(u < padd.nsplit ? u : 0) * padd.split_stride;
                    a0[PARTS ? it : 0][u] = *(const float4*)q;
                    a1[PARTS ? it : 0][u] = *(const float4*)(q + 4);
                }
            }
        }
    }
    const float p_amax = amax_from_lanes(p_amax_lane);

    // ---- arithmetic
    const float rl = rbf(rl_raw), xl = rbf(xl_raw), bl = rbf(bl_raw);
    const float p_inv_a = has_parts ? 1.0f / scale_from_amax(p_amax) : 0.f;
    float v[NV][8];
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int c = (threadIdx.x + it * 256) * 8;
        if (c < cols) {
            const uint32_t xw[4] = {xv[it].x, xv[it].y, xv[it].z, xv[it].w};
#pragma unroll
            for (int j = 0; j < 4; j++) v[it][2 * j] = bf16_lo(xw[j]), v[it][2 * j + 1] = bf16_hi(xw[j]);
            if (add) {
                const uint32_t aw[4] = {av[it].x, av[it].y, av[it].z, av[it].w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v[it][2 * j] = rbf(v[it][2 * j] + bf16_lo(aw[j]));
                    v[it][2 * j + 1] = rbf(v[it][2 * j + 1] + bf16_hi(aw[j]));
                }
            }
            if (has_parts) {
                float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
                // the sums keep the split order
#pragma unroll
                for (int u = 0; u < 8; u++) {
                    if (u < padd.nsplit) {
                        acc8[0] += a0[PARTS ? it : 0][u].x, acc8[1] += a0[PARTS ? it : 0][u].y, acc8[2] += a0[PARTS ? it : 0][u].z, acc8[3] += a0[PARTS ? it : 0][u].w;
                        acc8[4] += a1[PARTS ? it : 0][u].x, acc8[5] += a1[PARTS ? it : 0][u].y, acc8[6] += a1[PARTS ? it : 0][u].z, acc8[7] += a1[PARTS ? it : 0][u].w;
                    }
                }
                // splits beyond the first eight: again eight at a time, loads first
                const float* pp = padd.parts + (size_t)blockIdx.x * padd.ld + c;
                for (int sp0 = 8; sp0 < padd.nsplit; sp0 += 8) {
                    float4 b0[8], b1[8];
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        const float* q = pp + (size_t)(sp0 + u < padd.nsplit ? sp0 + u : sp0) * padd.split_stride;
                        b0[u] = *(const float4*)q;
                        b1[u] = *(const float4*)(q + 4);
                    }
#pragma unroll
                    for (int u = 0; u < 8; u++) {
                        if (sp0 + u < padd.nsplit) {
                            acc8[0] += b0[u].x, acc8[1] += b0[u].y, acc8[2] += b0[u].z, acc8[3] += b0[u].w;
                            acc8[4] += b1[u].x, acc8[5] += b1[u].y, acc8[6] += b1[u].z, acc8[7] += b1[u].w;
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < 8; j++) v[it][j] = rbf(v[it][j] + rbf((acc8[j] * p_inv_a) * p_inv_b));
            }
            if (backout_save)
                *(uint4*)(backout_save + base + c) = make_uint4(pack_bf16(v[it][0], v[it][1]), pack_bf16(v[it][2], v[it][3]),
                                                                pack_bf16(v[it][4], v[it][5]), pack_bf16(v[it][6], v[it][7]));
            const uint32_t zw[4] = {zv[it].x, zv[it].y, zv[it].z, zv[it].w};
            if (resid_lambda) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v[it][2 * j] = rbf(rbf(rl * v[it][2 * j]) + rbf(xl * bf16_lo(zw[j])));
                    v[it][2 * j + 1] = rbf(rbf(rl * v[it][2 * j + 1]) + rbf(xl * bf16_hi(zw[j])));
                }
            } else if (backout_lambda) {
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    v[it][2 * j] = rbf(v[it][2 * j] - rbf(bl * bf16_lo(zw[j])));
                    v[it][2 * j + 1] = rbf(v[it][2 * j + 1] - rbf(bl * bf16_hi(zw[j])));
                }
            }
            if (writes_x)
                *(uint4*)(x + base + c) = make_uint4(pack_bf16(v[it][0], v[it][1]), pack_bf16(v[it][2], v[it][3]),
                                                     pack_bf16(v[it][4], v[it][5]), pack_bf16(v[it][6], v[it][7]));
#pragma unroll
            for (int j = 0; j < 8; j++) ss += v[it][j] * v[it][j];
        }
    }
    ss = block_sum<4>(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)cols + RMS_EPS);
    float am = 0.f;
#pragma unroll
    for (int it = 0; it < NV; it++) {
        const int c = (threadIdx.x + it * 256) * 8;
        if (c < cols) {
            uint32_t o[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                o[j] = pack_bf16(v[it][2 * j] * rstd, v[it][2 * j + 1] * rstd);
                am = amax_fold(amax_fold(am, bf16_lo(o[j])), bf16_hi(o[j]));
            }
            *(uint4*)(xn_out + base + c) = make_uint4(o[0], o[1], o[2], o[3]);
        }
    }
    block_amax_commit(am, amax_ws, red);
    // the row's cache position, advanced here when this is the last kernel of a decode step that reads no positions any more
    if (bump && threadIdx.x == 0) bump[blockIdx.x] += bump_by;
}

// out = relu(h)^2, elementwise bf16, plus amax (gpt.py:139)
__global__ __launch_bounds__(256) void relu2_kernel(const bf16_t* __restrict__ h, bf16_t* __restrict__ out, int64_t n,
                                                    uint32_t* __restrict__ amax_ws) {
    __shared__ float red[8];
    float am = 0.f;
    const int64_t nvec = n / 8;
    for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < nvec; i += (int64_t)gridDim.x * blockDim.x) {
        uint4 v = ((const uint4*)h)[i];
        uint32_t w[4] = {v.x, v.y, v.z, v.w}, o[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            float a = relu_keep_nan(bf16_lo(w[j])), b = relu_keep_nan(bf16_hi(w[j]));
            a = rbf(a * a), b = rbf(b * b);
            am = amax_join(amax_join(am, a), b);
            o[j] = pack_bf16(a, b);
        }
        ((uint4*)out)[i] = make_uint4(o[0], o[1], o[2], o[3]);
    }
    if (blockIdx.x == 0)
        for (int64_t i = nvec * 8 + threadIdx.x; i < n; i += blockDim.x) {
            float a = relu_keep_nan(bf16_to_f32(h[i]));
            a = rbf(a * a);
            am = amax_join(am, a);
            out[i] = f32_to_bf16(a);
        }
    block_amax_commit(am, amax_ws, red);
}

// ------------------------------------------------------------------------------------------------
// One wave per (token, head) of the fused q|k|v projection output; lane l owns dims l and l+64, which
// is exactly one rotary pair.  head_dim is fixed at 128.
//   q heads: rotary -> rms_norm over D -> *1.2 -> q_out[token, h, :]
//   k heads: same -> k_cache[b, pos+t, h, :]
//   v heads: v + 3*sigmoid(W_g . xn[:12])[h] * ve[idx, h, :] (if the layer has a value embedding) -> v_cache
// (gpt.py:89-104, flash_attention.py:167-170)
__global__ __launch_bounds__(256) void qkv_rope_append_kernel(NcRopeSrc r, const int32_t* __restrict__ cache_seqlens,
                                                              bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                                                              bf16_t* __restrict__ q_out, int T, int H, int Hkv, int Tmax, int total_waves) {
    const int lane = threadIdx.x & 63;
    const int gw = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (gw >= total_waves) return;
    const int heads = H + 2 * Hkv;
    const int token = gw / heads, hh = gw % heads;
    const int b = token / T, t = token % T;
    const int pos = cache_seqlens[b] + t;
    float y1, y2;
    rope_head(r, token, pos, hh, H, Hkv, lane, y1, y2);
    bf16_t* dst;
    if (hh < H) dst = q_out + ((size_t)token * H + hh) * 128;
    else {
        if (pos < 0 || pos >= Tmax) return;
        const bool is_k = hh < H + Hkv;
        dst = (is_k ? k_cache : v_cache) + (((size_t)b * Tmax + pos) * Hkv + (is_k ? hh - H : hh - H - Hkv)) * 128;
    }
    dst[lane] = f32_to_bf16(y1);
    dst[lane + 64] = f32_to_bf16(y2);
}

// The same for many tokens (prefill), reading the bf16 output of the q|k|v linear: eight lanes share a head, each holding eight
// consecutive elements of its first half and the eight they pair with in the second half (element j rotates with j + 64), all
// accesses 16 bytes wide; the mean of squares of the QK-norm is a sum over the 8 lanes.  Same rounding points as rope_head_finish.
__global__ __launch_bounds__(256) void qkv_rope_append_vec_kernel(NcRopeSrc r, const int32_t* __restrict__ cache_seqlens,
                                                                  bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                                                                  bf16_t* __restrict__ q_out, int T, int H, int Hkv, int Tmax, int total_units) {
    const int part = threadIdx.x & 7;
    const int unit = blockIdx.x * 32 + (threadIdx.x >> 3);
    const bool live = unit < total_units;
    const int heads = H + 2 * Hkv;
    const int u = live ? unit : total_units - 1;             // idle lanes shadow the last unit (the lane shuffles below need every lane)
    const int token = u / heads, hh = u % heads;
    const int b = token / T, t = token % T;
    const int pos = cache_seqlens[b] + t;
    const bf16_t* src = r.qkv + (size_t)token * r.ld_qkv + (size_t)hh * 128 + part * 8;
    const uint4 xa = *(const uint4*)src, xb = *(const uint4*)(src + 64);
    const uint32_t wa[4] = {xa.x, xa.y, xa.z, xa.w}, wb[4] = {xb.x, xb.y, xb.z, xb.w};
    float x1[8], x2[8], o1[8], o2[8];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        x1[2 * j] = bf16_lo(wa[j]), x1[2 * j + 1] = bf16_hi(wa[j]);
        x2[2 * j] = bf16_lo(wb[j]), x2[2 * j + 1] = bf16_hi(wb[j]);
    }
    if (hh < H + Hkv) {
        const int rp = pos < r.rope_len ? (pos < 0 ? 0 : pos) : r.rope_len - 1;
        const uint4 cv = *(const uint4*)(r.cos_t + (size_t)rp * 64 + part * 8), sv = *(const uint4*)(r.sin_t + (size_t)rp * 64 + part * 8);
        const uint32_t cw[4] = {cv.x, cv.y, cv.z, cv.w}, sw[4] = {sv.x, sv.y, sv.z, sv.w};
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float c = (e & 1) ? bf16_hi(cw[e >> 1]) : bf16_lo(cw[e >> 1]);
            const float sn = (e & 1) ? bf16_hi(sw[e >> 1]) : bf16_lo(sw[e >> 1]);
            o1[e] = rbf(rbf(x1[e] * c) + rbf(x2[e] * sn));
            o2[e] = rbf(rbf(x1[e] * (-sn)) + rbf(x2[e] * c));
            ss += o1[e] * o1[e] + o2[e] * o2[e];
        }
        ss += __shfl_xor(ss, 1);
        ss += __shfl_xor(ss, 2);
        ss += __shfl_xor(ss, 4);
        const float rstd = 1.0f / sqrtf(ss / 128.0f + RMS_EPS);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            o1[e] = rbf(rbf(o1[e] * rstd) * 1.2f);
            o2[e] = rbf(rbf(o2[e] * rstd) * 1.2f);
        }
    } else {
#pragma unroll
        for (int e = 0; e < 8; e++) o1[e] = x1[e], o2[e] = x2[e];
        if (r.ve_table) {
            const int hv = hh - H - Hkv;
            int64_t tok = r.idx[token];
            if (tok < 0 || tok >= r.vocab_rows) tok = 0;
            const bf16_t* ve = r.ve_table + ((size_t)tok * Hkv + hv) * 128 + part * 8;
            const uint4 va = *(const uint4*)ve, vb = *(const uint4*)(ve + 64);
            const bf16_t* xg = r.xn + (size_t)token * r.ld_xn;
            float dot = 0.f;
#pragma unroll
            for (int c = 0; c < 12; c++) dot += bf16_to_f32(xg[c]) * rbf(r.ve_gate_w[hv * 12 + c]);
            const float gate = rbf(3.0f * rbf(sigmoidf_(rbf(dot))));
            const uint32_t ea[4] = {va.x, va.y, va.z, va.w}, eb[4] = {vb.x, vb.y, vb.z, vb.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v1 = (e & 1) ? bf16_hi(ea[e >> 1]) : bf16_lo(ea[e >> 1]);
                const float v2 = (e & 1) ? bf16_hi(eb[e >> 1]) : bf16_lo(eb[e >> 1]);
                o1[e] = rbf(o1[e] + rbf(gate * v1));
                o2[e] = rbf(o2[e] + rbf(gate * v2));
            }
        }
    }
    if (!live) return;
    bf16_t* dst;
    if (hh < H) dst = q_out + ((size_t)token * H + hh) * 128;
    else {
        if (pos < 0 || pos >= Tmax) return;
        const bool is_k = hh < H + Hkv;
        dst = (is_k ? k_cache : v_cache) + (((size_t)b * Tmax + pos) * Hkv + (is_k ? hh - H : hh - H - Hkv)) * 128;
    }
    dst += part * 8;
    *(uint4*)dst = make_uint4(pack_bf16(o1[0], o1[1]), pack_bf16(o1[2], o1[3]), pack_bf16(o1[4], o1[5]), pack_bf16(o1[6], o1[7]));
    *(uint4*)(dst + 64) = make_uint4(pack_bf16(o2[0], o2[1]), pack_bf16(o2[2], o2[3]), pack_bf16(o2[4], o2[5]), pack_bf16(o2[6], o2[7]));
}

// ------------------------------------------------------------------------------------------------
// KVCache.prefill (nanochat/engine.py:123-137): the first n positions of every (layer, row) of a source cache go to
// every row of a destination cache with a longer time axis; a one-row source is broadcast over the rows.  Each
// workgroup reads its 16 KB of a source (layer, row) once and writes it to all destination rows with streaming stores.
__global__ __launch_bounds__(256) void kv_prefill_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t vec_per_row,
                                                              size_t src_row_stride, size_t dst_row_stride, int src_rows, int dst_rows) {
    const int layer = blockIdx.y;
    // piece i of a thread is vector v0 + 256 i: every load and store instruction of a wave covers 1 KB of consecutive bytes
    const size_t v0 = (size_t)blockIdx.x * 1024 + threadIdx.x;
    const int b_first = src_rows == 1 ? 0 : blockIdx.z, b_last = src_rows == 1 ? dst_rows : blockIdx.z + 1;
    const uint4* sp = src + ((size_t)layer * src_rows + (src_rows == 1 ? 0 : blockIdx.z)) * src_row_stride;
    v4i r[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (v0 + 256 * i < vec_per_row) r[i] = *(const v4i*)(sp + v0 + 256 * i);
    for (int b = b_first; b < b_last; b++) {
        uint4* dp = dst + ((size_t)layer * dst_rows + b) * dst_row_stride;
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (v0 + 256 * i < vec_per_row) __builtin_nontemporal_store(r[i], (v4i*)(dp + v0 + 256 * i));
    }
}

int nc_launch_kv_prefill_copy(const void* src, void* dst, int layers, int src_rows, int dst_rows, int src_tmax, int dst_tmax,
                              int n_tokens, int token_bytes, hipStream_t s) {
    NC_CHECK_ARG(src && dst, "kv_prefill_copy: null pointer");
    NC_CHECK_ARG(layers > 0 && dst_rows > 0 && (src_rows == 1 || src_rows == dst_rows), "kv_prefill_copy: source rows must be 1 or match");
    NC_CHECK_ARG(n_tokens >= 0 && n_tokens <= src_tmax && n_tokens <= dst_tmax, "kv_prefill_copy: %d tokens do not fit (%d -> %d)", n_tokens,
                 src_tmax, dst_tmax);
    NC_CHECK_ARG(token_bytes > 0 && token_bytes % 16 == 0 && (((uintptr_t)src | (uintptr_t)dst) & 15) == 0,
                 "kv_prefill_copy: token size and pointers must be multiples of 16 bytes");
    NC_CHECK_ARG(layers <= 65535 && dst_rows <= 65535, "kv_prefill_copy: more than 65535 layers or rows");
    if (n_tokens == 0) return 0;
    const size_t vec_per_row = (size_t)n_tokens * token_bytes / 16;
    const size_t gx = (vec_per_row + 1023) / 1024;
    NC_CHECK_ARG(gx <= 0x7fffffff, "kv_prefill_copy: row too long");
    NcProfScope prof(3, 0.0, s);
    hipLaunchKernelGGL(kv_prefill_copy_kernel, dim3((unsigned)gx, layers, src_rows == 1 ? 1 : dst_rows), dim3(256), 0, s, (const uint4*)src,
                       (uint4*)dst, vec_per_row, (size_t)src_tmax * token_bytes / 16, (size_t)dst_tmax * token_bytes / 16, src_rows, dst_rows);
    NC_CHECK_LAUNCH("kv_prefill_copy");
    return 0;
}

// ------------------------------------------------------------------------------------------------
static bool row_args_ok(int rows, int cols) { return rows >= 0 && cols > 0 && cols <= 16384; }

int nc_launch_rmsnorm(const bf16_t* x, bf16_t* out, int rows, int cols, uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(x && out, "rmsnorm: null pointer");
    NC_CHECK_ARG(row_args_ok(rows, cols), "rmsnorm: bad shape rows=%d cols=%d (cols <= 16384)", rows, cols);
    // the mix kernel with no residual work never writes x
    return nc_launch_mix_norm(const_cast<bf16_t*>(x), nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, out, rows, cols,
                              amax_ws, s);
}

int nc_launch_embed_norm_smear(const int64_t* idx, const bf16_t* wte, const float* smear_w, const float* smear_lambda,
                               const bf16_t* prev_in, bf16_t* prev_out, bf16_t* x_out, bf16_t* x0_out, int B, int T, int E,
                               int vocab_rows, uint32_t* clear_words, int n_clear, hipStream_t s) {
    NC_CHECK_ARG(idx && wte && smear_w && smear_lambda && prev_out && x_out, "embed_norm_smear: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0 && E >= 24 && E <= 8192, "embed_norm_smear: bad shape B=%d T=%d E=%d", B, T, E);
    NcProfScope prof(3, 4.0 * B * T * E, s);
    const bool vec = T == 1 && E % 8 == 0 && E <= 2048 &&
                     (((uintptr_t)wte | (uintptr_t)prev_in | (uintptr_t)prev_out | (uintptr_t)x_out | (uintptr_t)x0_out) & 15) == 0;
    if (vec)
        hipLaunchKernelGGL(embed_norm_smear_decode_kernel, dim3(B), dim3(256), 0, s, idx, wte, smear_w, smear_lambda, prev_in, prev_out,
                           x_out, x0_out, E, vocab_rows, clear_words, clear_words ? n_clear : 0);
    else
        hipLaunchKernelGGL(embed_norm_smear_kernel, dim3(B * T), dim3(256), 2 * E * sizeof(float), s, idx, wte, smear_w, smear_lambda,
                           prev_in, prev_out, x_out, x0_out, T, E, vocab_rows, clear_words, clear_words ? n_clear : 0);
    NC_CHECK_LAUNCH("embed_norm_smear");
    return 0;
}

static int launch_mix_norm_impl(bf16_t* x, const bf16_t* add, NcPartialSrc padd, const bf16_t* x0, const float* resid_lambda,
                                const float* x0_lambda, const float* backout_lambda, const bf16_t* backout_src, bf16_t* backout_save,
                                bf16_t* xn_out, int rows, int cols, uint32_t* amax_ws, hipStream_t s, int32_t* bump, int bump_by) {
    NC_CHECK_ARG(x && xn_out, "mix_norm: null pointer");
    NC_CHECK_ARG(row_args_ok(rows, cols), "mix_norm: bad shape rows=%d cols=%d", rows, cols);
    NC_CHECK_ARG(!resid_lambda || (x0 && x0_lambda), "mix_norm: the residual mix needs x0 and x0_lambda");
    NC_CHECK_ARG(!backout_lambda || backout_src, "mix_norm: backout needs its source rows");
    NC_CHECK_ARG(!(resid_lambda && backout_lambda), "mix_norm: residual mix and backout are exclusive");
    NC_CHECK_ARG(!(add && padd.parts), "mix_norm: give the added tensor either as bf16 or as partials");
    if (rows == 0) return 0;
    NcProfScope prof(3, 8.0 * rows * cols, s);
    const bool aligned = cols % 8 == 0 && (((uintptr_t)x | (uintptr_t)xn_out | (uintptr_t)add | (uintptr_t)x0 | (uintptr_t)backout_src |
                                            (uintptr_t)backout_save | (uintptr_t)padd.parts) & 15) == 0 && padd.ld % 4 == 0 &&
                         padd.split_stride % 4 == 0;
#define MIX_ARGS x, add, padd, x0, resid_lambda, x0_lambda, backout_lambda, backout_src, backout_save, xn_out, cols, amax_ws, bump, bump_by
#define MIX_LAUNCH(NVV)                                                                                                  \
    do {                                                                                                                 \
        if (padd.parts) hipLaunchKernelGGL((mix_norm_vec_kernel<NVV, true>), dim3(rows), dim3(256), 0, s, MIX_ARGS);      \
        else hipLaunchKernelGGL((mix_norm_vec_kernel<NVV, false>), dim3(rows), dim3(256), 0, s, MIX_ARGS);                \
    } while (0)
    if (aligned && cols <= 2048) MIX_LAUNCH(1);
    else if (aligned && cols <= 4096) MIX_LAUNCH(2);
    else if (aligned && cols <= 8192) MIX_LAUNCH(4);
    else {
        NC_CHECK_ARG(!padd.parts && !bump, "mix_norm: partial-sum input and the position advance need cols %% 8 == 0, cols <= 8192 and 16-byte alignment");
        hipLaunchKernelGGL(mix_norm_kernel, dim3(rows), dim3(256), cols * sizeof(float), s, x, add, x0, resid_lambda, x0_lambda,
                           backout_lambda, backout_src, backout_save, xn_out, cols, amax_ws);
    }
#undef MIX_LAUNCH
#undef MIX_ARGS
    NC_CHECK_LAUNCH("mix_norm");
    return 0;
}

int nc_launch_mix_norm(bf16_t* x, const bf16_t* add, const bf16_t* x0, const float* resid_lambda, const float* x0_lambda,
                       const float* backout_lambda, const bf16_t* backout_src, bf16_t* backout_save, bf16_t* xn_out,
                       int rows, int cols, uint32_t* amax_ws, hipStream_t s, int32_t* bump, int bump_by) {
    NcPartialSrc none{nullptr, 0, 0, 0, nullptr, nullptr, 0, 0};
    return launch_mix_norm_impl(x, add, none, x0, resid_lambda, x0_lambda, backout_lambda, backout_src, backout_save, xn_out, rows,
                                cols, amax_ws, s, bump, bump_by);
}

int nc_launch_mix_norm_p(bf16_t* x, NcPartialSrc add, const bf16_t* x0, const float* resid_lambda, const float* x0_lambda,
                         const float* backout_lambda, const bf16_t* backout_src, bf16_t* backout_save, bf16_t* xn_out,
                         int rows, int cols, uint32_t* amax_ws, hipStream_t s, int32_t* bump, int bump_by) {
    NC_CHECK_ARG(!add.parts || (add.nsplit >= 1 && add.a_amax && add.inv_b && add.ld >= cols), "mix_norm: bad partial-sum source");
    return launch_mix_norm_impl(x, nullptr, add, x0, resid_lambda, x0_lambda, backout_lambda, backout_src, backout_save, xn_out, rows,
                                cols, amax_ws, s, bump, bump_by);
}

int nc_launch_relu2(const bf16_t* h, bf16_t* out, int64_t n, uint32_t* amax_ws, hipStream_t s) {
    NC_CHECK_ARG(h && out && n >= 0, "relu2: bad arguments");
    NC_CHECK_ARG(((uintptr_t)h & 15) == 0 && ((uintptr_t)out & 15) == 0, "relu2: pointers must be 16-byte aligned");
    int64_t g = (n / 8 + 255) / 256;
    if (g < 1) g = 1;
    if (g > 2048) g = 2048;
    NcProfScope prof(3, 4.0 * n, s);
    hipLaunchKernelGGL(relu2_kernel, dim3((int)g), dim3(256), 0, s, h, out, n, amax_ws);
    NC_CHECK_LAUNCH("relu2");
    return 0;
}

static int launch_rope_impl(const bf16_t* qkv, int ld_qkv, NcPartialSrc pq, const bf16_t* xn, int ld_xn, const int64_t* idx,
                            const bf16_t* ve_table, const float* ve_gate_w, const bf16_t* cos, const bf16_t* sin, int rope_len,
                            const int32_t* cache_seqlens, bf16_t* k_cache, bf16_t* v_cache, bf16_t* q_out, int B, int T, int H, int Hkv,
                            int Tmax, int vocab_rows, hipStream_t s) {
    NC_CHECK_ARG((qkv || pq.parts) && cos && sin && cache_seqlens && k_cache && v_cache && q_out, "qkv_rope_append: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0 && H > 0 && Hkv > 0 && H % Hkv == 0 && Tmax > 0 && rope_len > 0, "qkv_rope_append: bad shape");
    NC_CHECK_ARG((pq.parts ? pq.ld : ld_qkv) >= (H + 2 * Hkv) * 128, "qkv_rope_append: row stride too small (head_dim is fixed at 128)");
    NC_CHECK_ARG(!ve_table || (ve_gate_w && xn && idx && ld_xn >= 12), "qkv_rope_append: value embedding needs gate weights, xn and idx");
    const int total = B * T * (H + 2 * Hkv);
    NcProfScope prof(3, 4.0 * total * 128, s);
    const NcRopeSrc r{qkv, ld_qkv, pq, xn, ld_xn, idx, ve_table, ve_gate_w, cos, sin, rope_len, vocab_rows, nullptr, nullptr};
    // many tokens of finished bf16 rows: the 16-byte-wide kernel (8 lanes per head); a few tokens, or rows still in split partials:
    // one wave per head
    const bool wide = qkv && total >= 2048 && ld_qkv % 8 == 0 && ld_xn % 8 == 0 &&
                      ((((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)q_out | (uintptr_t)cos | (uintptr_t)sin | (uintptr_t)ve_table) & 15) == 0);
    if (wide)
        hipLaunchKernelGGL(qkv_rope_append_vec_kernel, dim3((total + 31) / 32), dim3(256), 0, s, r, cache_seqlens, k_cache, v_cache, q_out, T, H,
                           Hkv, Tmax, total);
    else
        hipLaunchKernelGGL(qkv_rope_append_kernel, dim3((total + 3) / 4), dim3(256), 0, s, r, cache_seqlens, k_cache, v_cache, q_out, T, H,
                           Hkv, Tmax, total);
    NC_CHECK_LAUNCH("qkv_rope_append");
    return 0;
}

int nc_launch_qkv_rope_append(const bf16_t* qkv, int ld_qkv, const bf16_t* xn, int ld_xn, const int64_t* idx,
                              const bf16_t* ve_table, const float* ve_gate_w, const bf16_t* cos, const bf16_t* sin,
                              int rope_len, const int32_t* cache_seqlens, bf16_t* k_cache, bf16_t* v_cache, bf16_t* q_out,
                              int B, int T, int H, int Hkv, int Tmax, int vocab_rows, hipStream_t s) {
    NcPartialSrc none{nullptr, 0, 0, 0, nullptr, nullptr, 0, 0};
    return launch_rope_impl(qkv, ld_qkv, none, xn, ld_xn, idx, ve_table, ve_gate_w, cos, sin, rope_len, cache_seqlens, k_cache, v_cache,
                            q_out, B, T, H, Hkv, Tmax, vocab_rows, s);
}

int nc_launch_qkv_rope_append_p(NcPartialSrc qkv_parts, const bf16_t* xn, int ld_xn, const int64_t* idx,
                                const bf16_t* ve_table, const float* ve_gate_w, const bf16_t* cos, const bf16_t* sin,
                                int rope_len, const int32_t* cache_seqlens, bf16_t* k_cache, bf16_t* v_cache, bf16_t* q_out,
                                int B, int T, int H, int Hkv, int Tmax, int vocab_rows, hipStream_t s) {
    NC_CHECK_ARG(qkv_parts.parts && qkv_parts.nsplit >= 1 && qkv_parts.a_amax && qkv_parts.inv_b, "qkv_rope_append: bad partial-sum source");
    return launch_rope_impl(nullptr, 0, qkv_parts, xn, ld_xn, idx, ve_table, ve_gate_w, cos, sin, rope_len, cache_seqlens, k_cache,
                            v_cache, q_out, B, T, H, Hkv, Tmax, vocab_rows, s);
}
