// Host-side sequencing of one GPT.forward(idx, kv_cache=...) on a stream: the native replacement of the
// Python loop at nanochat/gpt.py:459-524 (and of the module calls it makes into gpt.py:84-153 and
// fp8.py:202-213).  One call enqueues every kernel of the step; no host synchronisation, no allocation.
//
// Per layer, decode (M = B*T <= 128 rows), 8 launches, each making a single dependent trip to memory:
//   mix_norm            x += mlp_out(prev) [read from split partials]; x = rl*x + xl*x0; xn = norm(x); amax(xn)
//   linear q|k|v        quantize xn inside the GEMM; K split over workgroups           -> fp32 partials
//   attention           each (row, kv head) workgroup first sums its heads' partials (three weight scales), applies
//                       rotary, QK-norm, gain and the VE gate, appends key and value to the cache, then attends over
//                       the cache; amax(y)                                             -> y
//                       (small batches, where attention is split over several workgroups per head, and T > 1 keep the
//                       stand-alone qkv_rope_append kernel in front)
//   linear c_proj       quantize y inside                                              -> partials
//   mix_norm            x += o [from partials]; xn = norm(x); amax(xn)
//   linear c_fc         quantize xn inside                                             -> partials
//   finish_partials     sum, scale, relu^2, amax                                       -> h2
//   linear mlp c_proj   quantize h2 inside                                             -> partials (added by the next mix_norm)
// Prefill (M > 128) uses the explicit convert kernel and the tiled GEMM instead of the fused small-M linear.
//
// Workspace (carved from the caller's buffer, 256-byte aligned pieces), M = B*T rows:
//   x, x0, xn, xb, o      bf16 [M,E]        residual stream, its initial value, normed rows, backout, GEMM out
//   qkv                   bf16 [M,(H+2Hkv)*128]
//   qh, y                 bf16 [M,H*128]    rotated queries, attention output
//   h, h2                 bf16 [M,4E]       c_fc output (prefill only), relu^2
//   a8                    u8   [M,4E]       quantized activations (prefill only)
//   xl                    bf16 [B,E]        last-position rows (last_only lm_head at T > 1)
//   inv                   fp32 [4L+1]       activation inverse scales (prefill only)
//   zeroed                u32               amax sites [4L+1] x 8 slots on separate lines | attention split counters,
//                                           cleared by the embedding kernel at the start of the call
//   gemm_parts, attn_parts                  split partials of the small-M linears and of attention
#include <stdio.h>
#include "../../include/nanochat_amd.h"
#include "nc_common.h"
#include "nc_kernels.h"
#include "nc_rope.h"

#define TRY(call)              \
    do {                       \
        int rc__ = (call);     \
        if (rc__) return rc__; \
    } while (0)

// Reading a shared prompt once for all rows costs two more launches per layer (the stand-alone rotary kernel and the shared-keys kernel,
// ~12-14 us together with the merge) and saves the per-row streaming of the shared keys the layer sees: rows x kv heads x keys x 512
// bytes at ~6 TB/s.  It is taken when that is at least ~14 us: 164 000 (row, kv head, key) units -- 197 shared keys at 64 rows of 13
// heads (a full-context layer always; a 512-key window until it has moved most of the way out of the prompt), 394 at 32 rows.
// (measured through the harness at d26, 1792-token prompt: 8 / 16 / 32 rows 1.38 / 1.58 / 2.14 -> 1.30 / 1.43 / 1.79 ms per step)
#define NC_SHARED_MIN_ROW_HEADS 64
#define NC_SHARED_MIN_KEYS 128
#define NC_SHARED_MIN_UNITS 164000L

namespace {
struct Carver {
    uint8_t* base;
    size_t off = 0;
    explicit Carver(void* p) : base((uint8_t*)p) {}
    template <typename T>
    T* take(size_t count) {
        off = (off + 255) & ~(size_t)255;
        T* r = base ? (T*)(base + off) : nullptr;
        off += count * sizeof(T);
        return r;
    }
};

struct Workspace {
    bf16_t *x, *x0, *xn, *xb, *o, *qkv, *qh, *y, *h, *h2, *xl;
    bf16_t* x2;                // second residual-stream buffer of the one- and two-row decode step (see fused_rows())
    uint8_t* a8;
    float* inv;
    uint32_t *amax, *attn_counters;
    // handle of amax site i (tagged: NC_AMAX_SLOTS words on separate lines, see amax_read / amax_publish)
    uint32_t* site(int i) const { return nc_amax_slotted(amax + (size_t)i * NC_AMAX_SLOTS * NC_AMAX_STRIDE); }
    int zero_words;
    uint8_t *gemm_parts, *gemm_parts2, *attn_parts, *shared_parts;
    size_t gemm_part_bytes, attn_part_bytes, shared_part_bytes;
    size_t total;
};

// One or two rows (a chat session's decode step): the residual/norm passes and the relu^2 pass are folded into the linears that consume
// them (NcRowRecipe), five launches per layer instead of eight.  Each such linear reads its input recipe's partial sums from one
// buffer and writes its own into the other, and the residual stream alternates between two buffers in the same way, because the
// workgroups of one launch must not overwrite what their neighbours still read.
bool fused_rows(const nc_model_desc* m, int M) {
    const int E = m->n_embd, qkv_w = (m->n_head + 2 * m->n_kv_head) * 128;
    if (M > NC_RECIPE_MAX_ROWS || E > 2048 || 4 * E > NC_RECIPE_MAX_K || E % 8 != 0) return false;
    // every linear of a layer must leave split partial sums (the recipe of the next one reads them)
    return nc_gemm_decode_splits(qkv_w, E) > 1 && nc_gemm_decode_splits(E, m->n_head * 128) > 1 && nc_gemm_decode_splits(4 * E, E) > 1 &&
           nc_gemm_decode_splits(E, 4 * E) > 1;
}

Workspace carve(const nc_model_desc* m, int B, int T, void* base) {
    const size_t M = (size_t)B * T, E = m->n_embd;
    const size_t qkv_w = (size_t)(m->n_head + 2 * m->n_kv_head) * 128;
    const bool small = M <= 128;
    Carver c(base);
    Workspace w;
    w.x = c.take<bf16_t>(M * E);
    w.x2 = c.take<bf16_t>(fused_rows(m, (int)M) ? M * E : 0);
    w.x0 = c.take<bf16_t>(M * E);
    w.xn = c.take<bf16_t>(M * E);
    w.xb = c.take<bf16_t>(M * E);
    w.o = c.take<bf16_t>(M * E);
    w.qkv = c.take<bf16_t>(M * qkv_w);
    w.qh = c.take<bf16_t>(M * m->n_head * 128);
    w.y = c.take<bf16_t>(M * m->n_head * 128);
    w.h = c.take<bf16_t>(small ? 0 : M * 4 * E);
    w.h2 = c.take<bf16_t>(M * 4 * E);
    w.a8 = c.take<uint8_t>(small ? 0 : M * 4 * E);
    w.xl = c.take<bf16_t>((size_t)B * E);
    w.inv = c.take<float>(4 * (size_t)m->n_layer + 1);
    const size_t amax_words = (4 * (size_t)m->n_layer + 1) * NC_AMAX_SLOTS * NC_AMAX_STRIDE;     // one slotted site per FP8 linear input
    // attention split counters and partials only when some layer's launch really splits its keys over workgroups (never with 16 or
    // more queries per row, which take the matrix-core kernel, and never once rows x kv heads fill the chip); the cache length is not
    // known here, so each layer is sized for its whole window
    int max_splits = 1;
    if (T < 16)
        for (int i = 0; i < m->n_layer; i++) {
            const int sp = nc_attn_splits(B, T, m->n_kv_head, m->layers ? m->layers[i].window_left : -1, 1 << 30);
            max_splits = sp > max_splits ? sp : max_splits;
        }
    const size_t attn_words = max_splits > 1 ? nc_attn_counter_bytes(B, T, m->n_head) / 4 : 0;
    uint32_t* zero = c.take<uint32_t>(amax_words + attn_words);
    w.amax = zero;
    w.attn_counters = zero ? zero + amax_words : nullptr;
    w.zero_words = (int)(amax_words + attn_words);
    size_t gneed = 0;
    if (small) {
        const int shapes[5][2] = {{(int)qkv_w, (int)E}, {(int)E, m->n_head * 128}, {(int)(4 * E), (int)E}, {(int)E, (int)(4 * E)},
                                  {m->vocab_size, (int)E}};
        for (auto& sh : shapes) {
            const size_t n = nc_gemm_decode_partial_bytes_auto((int)M, sh[0], sh[1]);
            gneed = n > gneed ? n : gneed;
        }
    }
    w.gemm_part_bytes = gneed;
    w.gemm_parts = c.take<uint8_t>(gneed);
    w.gemm_parts2 = c.take<uint8_t>(fused_rows(m, (int)M) ? gneed : 0);
    w.attn_part_bytes = max_splits > 1 ? nc_attn_partial_bytes(B, T, m->n_head) / 16 * max_splits : 0;
    w.attn_parts = c.take<uint8_t>(w.attn_part_bytes);
    // partial results of the shared first part of the cache (rows that begin with one replicated prompt): whatever the shared length
    // turns out to be, the launch cuts it into at most as many chunks as a whole cache row would get
    w.shared_part_bytes = (T == 1 && (long)B * m->n_kv_head >= NC_SHARED_MIN_ROW_HEADS) ? nc_attn_shared_partial_bytes(B, m->n_head, m->n_kv_head, 1 << 20) : 0;
    w.shared_parts = c.take<uint8_t>(w.shared_part_bytes);
    w.total = (c.off + 255) & ~(size_t)255;
    return w;
}

NcGemmSegs one_seg(int n) { return NcGemmSegs{1, {n, 0, 0, 0}}; }

__global__ void gather_last_rows_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out, int T, int E) {
    const int b = blockIdx.x;
    const bf16_t* src = x + ((size_t)b * T + (T - 1)) * E;
    for (int c = threadIdx.x; c < E; c += blockDim.x) out[(size_t)b * E + c] = src[c];
}

const NcPartialSrc NO_PARTIALS{nullptr, 0, 0, 0, nullptr, nullptr, 0, 0};

int tap_copy(bf16_t* dst, const bf16_t* src, size_t elems, hipStream_t s) {
    const hipError_t e = hipMemcpyAsync(dst, src, elems * sizeof(bf16_t), hipMemcpyDeviceToDevice, s);
    if (e != hipSuccess) NC_FAIL(-2, "gpt_forward: tap copy failed: %s", hipGetErrorString(e));
    return 0;
}

// One FP8 linear on `rows` rows of bf16 input whose amax sits in slot `site`.  Small M: the result is either
// in `out` (single split: epilogue done in the GEMM) or described by *src (split partials for the consumer).
struct LinearRunner {
    const Workspace& w;
    hipStream_t s;
    // The same linear with its input rows made inside the kernel (one or two rows); the partial sums go to `parts_buf`.
    int run_recipe(const NcRowRecipe& recipe, int rows, int site, const uint8_t* w8, const float* inv_w, NcGemmSegs segs, int N, int K,
                   uint8_t* parts_buf, NcPartialSrc* src) const {
        int used = 1;
        const int want = nc_gemm_decode_splits(N, K);
        // (a single split would need the epilogue in the GEMM; every linear of a layer splits K, and the recipe path relies on it)
        NC_CHECK_ARG(want > 1, "gpt_forward: the fused small-batch step needs split linears (N=%d K=%d)", N, K);
        TRY(nc_launch_gemm_decode(nullptr, 1, nullptr, nullptr, w8, inv_w, segs, nullptr, 0, 0.f, nullptr, rows, N, K, N, (float*)parts_buf,
                                  w.gemm_part_bytes, want, &used, s, &recipe));
        *src = NcPartialSrc{(const float*)parts_buf, used, N, (size_t)rows * N, w.site(site), inv_w,
                            segs.nseg > 1 ? segs.end[0] : 0x7fffffff, segs.nseg > 2 ? segs.end[1] : 0x7fffffff};
        return 0;
    }
    int run(const bf16_t* in, int rows, int site, const uint8_t* w8, const float* inv_w, NcGemmSegs segs, void* out, int out_kind,
            float softcap, uint32_t* out_amax, int N, int K, int ldc, NcPartialSrc* src, uint8_t* parts_buf = nullptr) const {
        if (src) *src = NO_PARTIALS;
        uint8_t* const pbuf = parts_buf ? parts_buf : w.gemm_parts;
        if (rows <= 128) {
            int used = 1;
            TRY(nc_launch_gemm_decode(in, 1, w.site(site), nullptr, w8, inv_w, segs, out, out_kind, softcap, out_amax, rows, N, K, ldc,
                                      (float*)pbuf, w.gemm_part_bytes, src || out_kind == 2 ? 0 : 1, &used, s));
            if (used == 1) return 0;
            if (src) {
                *src = NcPartialSrc{(const float*)pbuf, used, N, (size_t)rows * N, w.site(site), inv_w,
                                    segs.nseg > 1 ? segs.end[0] : 0x7fffffff, segs.nseg > 2 ? segs.end[1] : 0x7fffffff};
                return 0;
            }
            return nc_launch_finish_partials((const float*)pbuf, used, w.site(site), nullptr, inv_w, segs, out, out_kind, softcap,
                                             out_amax, rows, N, ldc, s);
        }
        // large M: explicit convert pass, tiled GEMM; relu^2 (out_kind 2) is a separate kernel there
        TRY(nc_launch_convert_only(in, (int64_t)rows * K, w.a8, w.inv + site, w.site(site), s));
        if (out_kind == 2) {
            // relu^2 and its amax in the GEMM's epilogue; past the 32-bit buffer offsets, the plain-load kernel and a separate pass
            if ((long)rows * K < (1L << 31) && (long)N * K < (1L << 31))
                return nc_launch_gemm(w.a8, w8, w.inv + site, inv_w, segs, out, 2, 0.f, rows, N, K, ldc, 0, nullptr, 0, s, 0, out_amax);
            TRY(nc_launch_gemm(w.a8, w8, w.inv + site, inv_w, segs, w.h, 0, 0.f, rows, N, K, N, 0, nullptr, 0, s));
            return nc_launch_relu2(w.h, (bf16_t*)out, (int64_t)rows * N, out_amax, s);
        }
        return nc_launch_gemm(w.a8, w8, w.inv + site, inv_w, segs, out, out_kind, softcap, rows, N, K, ldc, 0, nullptr, 0, s);
    }
};
}  // namespace

extern "C" size_t nc_gpt_workspace_bytes(const nc_model_desc* model, int B, int T) {
    if (!model || B <= 0 || T <= 0) return 0;
    return carve(model, B, T, nullptr).total;
}

// tap_x (or nullptr): bf16 [L+1, M, E], slot i = the residual stream as layer i reads it (after the lambda mix, gpt.py:500), slot L = the
// final normalised rows (gpt.py:508).  tap_y (or nullptr): bf16 [L, M, H*128], the attention outputs before c_proj (gpt.py:113-124).
static int gpt_forward_impl(const nc_model_desc* m, const nc_cache_desc* kv, const int64_t* idx, int B, int T, float* logits_out,
                            int last_only, void* workspace, size_t workspace_bytes, bf16_t* tap_x, bf16_t* tap_y, hipStream_t s) {
    NC_CHECK_ARG(m && kv && idx && logits_out && workspace, "gpt_forward: null pointer");
    NC_CHECK_ARG(B > 0 && T > 0, "gpt_forward: bad batch/time B=%d T=%d", B, T);
    NC_CHECK_ARG(m->n_embd == m->n_head * 128, "gpt_forward: head_dim must be 128 (n_embd=%d n_head=%d)", m->n_embd, m->n_head);
    NC_CHECK_ARG(m->n_embd % 16 == 0 && m->n_embd >= 128, "gpt_forward: n_embd=%d must pass the FP8 filter", m->n_embd);
    NC_CHECK_ARG(kv->batch == B, "gpt_forward: cache batch %d != B %d", kv->batch, B);
    NC_CHECK_ARG(kv->k_cache && kv->v_cache && kv->cache_seqlens && kv->prev_out, "gpt_forward: cache pointers missing");
    NC_CHECK_ARG(((uintptr_t)workspace & 255) == 0, "gpt_forward: workspace must be 256-byte aligned");
    Workspace w = carve(m, B, T, workspace);
    NC_CHECK_ARG(workspace_bytes >= w.total, "gpt_forward: workspace of %zu bytes needed, %zu given", w.total, workspace_bytes);

    const int L = m->n_layer, E = m->n_embd, H = m->n_head, Hkv = m->n_kv_head, M = B * T;
    const int qkv_w = (H + 2 * Hkv) * 128;
    const size_t layer_elems = (size_t)B * kv->max_seq_len * Hkv * 128;
    const LinearRunner lin{w, s};
    int site = 0;   // amax / inv slot of the next FP8 linear input

    // x0 is the post-smear embedding; layer 0 reads it through both x and x0 (gpt.py:495,500)
    TRY(nc_launch_embed_norm_smear(idx, m->wte, m->smear_w, m->smear_lambda, kv->prev_in, kv->prev_out, w.x, w.x0, B, T, E,
                                   m->padded_vocab, w.amax, w.zero_words, s));

    // output of the previous MLP projection, still to be added into the residual stream: bf16 rows or split partials
    const bf16_t* pending_add = nullptr;
    NcPartialSrc pending_parts = NO_PARTIALS;
    auto mix = [&](const float* rl, const float* xl, const float* bl, const bf16_t* bsrc, bf16_t* save, uint32_t* amax,
                   int32_t* bump = nullptr, int bump_by = 0) -> int {
        if (pending_parts.parts)
            return nc_launch_mix_norm_p(w.x, pending_parts, w.x0, rl, xl, bl, bsrc, save, w.xn, M, E, amax, s, bump, bump_by);
        return nc_launch_mix_norm(w.x, pending_add, w.x0, rl, xl, bl, bsrc, save, w.xn, M, E, amax, s, bump, bump_by);
    };
    // (measured at d26, steps without a synchronisation in between: one row 1.30 -> 1.13 ms, two rows 1.37 -> 1.27 ms)
    const bool fused = T == 1 && fused_rows(m, M);
    bf16_t *xcur = w.x, *xalt = w.x2;            // fused step: the residual stream alternates between the two
    uint8_t *pin = w.gemm_parts, *pout = w.gemm_parts2;      // ... and so do the partial sums: pending_parts always sits in `pin`
    for (int i = 0; i < L && fused; i++) {
        const nc_layer_desc& ly = m->layers[i];
        NC_CHECK_ARG(ly.w_qkv && ly.inv_qkv && ly.w_attn_proj && ly.w_fc && ly.w_mlp_proj, "gpt_forward: layer %d has no FP8 weights", i);
        // q|k|v linear on rows it makes itself: x += mlp_out(prev layer); [save backout]; x = rl*x + xl*x0; xn = norm(x)
        NcRowRecipe mix1{};
        mix1.kind = 1, mix1.x_in = xcur, mix1.x_out = xalt, mix1.add = nullptr, mix1.padd = pending_parts, mix1.x0 = w.x0;
        mix1.resid_lambda = m->resid_lambdas + i, mix1.x0_lambda = m->x0_lambdas + i;
        mix1.save = (i > 0 && (i - 1) == L / 2) ? w.xb : nullptr, mix1.xn_out = w.xn, mix1.amax_out = w.site(site);
        NcGemmSegs qkv_segs{3, {H * 128, (H + Hkv) * 128, qkv_w, 0}};
        NcPartialSrc qsrc;
        TRY(lin.run_recipe(mix1, M, site, ly.w_qkv, ly.inv_qkv, qkv_segs, qkv_w, E, pout, &qsrc));
        { bf16_t* t = xcur; xcur = xalt; xalt = t; }
        { uint8_t* t = pin; pin = pout; pout = t; }          // the q|k|v partial sums are in `pin` now
        site++;
        if (tap_x) TRY(tap_copy(tap_x + (size_t)i * M * E, xcur, (size_t)M * E, s));
        bf16_t* kc = kv->k_cache + (size_t)i * layer_elems;
        bf16_t* vc = kv->v_cache + (size_t)i * layer_elems;
        const NcRopeSrc rope{nullptr, qkv_w, qsrc, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len, m->padded_vocab,
                             nullptr, nullptr};
        TRY(nc_launch_attention_fused(rope, kc, vc, kv->cache_seqlens, ly.window_left, w.y, B, H, Hkv, kv->max_seq_len, w.attn_counters,
                                      w.attn_parts, w.attn_part_bytes, w.site(site), 0, 1, s));
        if (tap_y) TRY(tap_copy(tap_y + (size_t)i * M * H * 128, w.y, (size_t)M * H * 128, s));
        // attention c_proj reads y as before; its partial sums go to the other buffer (the q|k|v ones are consumed by now)
        TRY(lin.run(w.y, M, site, ly.w_attn_proj, ly.inv_attn_proj, one_seg(E), w.o, 0, 0.f, nullptr, E, H * 128, E, &pending_parts, pout));
        NC_CHECK_ARG(pending_parts.parts, "gpt_forward: the fused small-batch step needs a split attention projection");
        { uint8_t* t = pin; pin = pout; pout = t; }
        site++;
        // c_fc on rows it makes itself: x += attn_out; xn = norm(x)
        NcRowRecipe mix2{};
        mix2.kind = 1, mix2.x_in = xcur, mix2.x_out = xalt, mix2.padd = pending_parts, mix2.xn_out = w.xn, mix2.amax_out = w.site(site);
        NcPartialSrc fsrc;
        TRY(lin.run_recipe(mix2, M, site, ly.w_fc, ly.inv_fc, one_seg(4 * E), 4 * E, E, pout, &fsrc));
        { bf16_t* t = xcur; xcur = xalt; xalt = t; }
        { uint8_t* t = pin; pin = pout; pout = t; }
        site++;
        // MLP projection on rows it makes itself: h2 = relu(c_fc(xn))^2
        NcRowRecipe act{};
        act.kind = 2, act.padd = fsrc, act.amax_out = w.site(site);
        TRY(lin.run_recipe(act, M, site, ly.w_mlp_proj, ly.inv_mlp_proj, one_seg(E), E, 4 * E, pout, &pending_parts));
        { uint8_t* t = pin; pin = pout; pout = t; }
        site++;
    }
    if (fused && xcur != w.x) {
        // the last pass below works on w.x
        const hipError_t e = hipMemcpyAsync(w.x, xcur, (size_t)M * E * sizeof(bf16_t), hipMemcpyDeviceToDevice, s);
        if (e != hipSuccess) NC_FAIL(-2, "gpt_forward: copy of the residual rows failed: %s", hipGetErrorString(e));
    }
    for (int i = 0; i < L && !fused; i++) {
        const nc_layer_desc& ly = m->layers[i];
        NC_CHECK_ARG(ly.w_qkv && ly.inv_qkv && ly.w_attn_proj && ly.w_fc && ly.w_mlp_proj, "gpt_forward: layer %d has no FP8 weights", i);
        // x += mlp_out(prev layer); [save backout]; x = rl*x + xl*x0; xn = norm(x)
        bf16_t* save = (i > 0 && (i - 1) == L / 2) ? w.xb : nullptr;
        TRY(mix(m->resid_lambdas + i, m->x0_lambdas + i, nullptr, nullptr, save, w.site(site)));
        if (tap_x) TRY(tap_copy(tap_x + (size_t)i * M * E, w.x, (size_t)M * E, s));
        // q|k|v = FP8 linear(xn): one activation quantization, three weight scales
        NcGemmSegs qkv_segs{3, {H * 128, (H + Hkv) * 128, qkv_w, 0}};
        NcPartialSrc qsrc;
        TRY(lin.run(w.xn, M, site, ly.w_qkv, ly.inv_qkv, qkv_segs, w.qkv, 0, 0.f, nullptr, qkv_w, E, qkv_w, &qsrc));
        site++;
        bf16_t* kc = kv->k_cache + (size_t)i * layer_elems;
        bf16_t* vc = kv->v_cache + (size_t)i * layer_elems;
        // rows that begin with one replicated prompt: a layer that sees a long stretch of it reads that stretch once for all rows
        bool shared_done = false;
        if (T == 1 && (long)B * Hkv >= NC_SHARED_MIN_ROW_HEADS && kv->shared_prefix > 0 && kv->uniform_pos >= kv->shared_prefix && w.shared_parts) {
            const int first_visible = ly.window_left < 0 ? 0 : (kv->uniform_pos - ly.window_left > 0 ? kv->uniform_pos - ly.window_left : 0);
            const int shared_visible = kv->shared_prefix - first_visible;
            if (shared_visible >= NC_SHARED_MIN_KEYS && (long)shared_visible * B * Hkv >= NC_SHARED_MIN_UNITS && kv->shared_prefix < kv->max_seq_len) {
                if (qsrc.parts)
                    TRY(nc_launch_qkv_rope_append_p(qsrc, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len,
                                                    kv->cache_seqlens, kc, vc, w.qh, B, T, H, Hkv, kv->max_seq_len, m->padded_vocab, s));
                else
                    TRY(nc_launch_qkv_rope_append(w.qkv, qkv_w, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len,
                                                  kv->cache_seqlens, kc, vc, w.qh, B, T, H, Hkv, kv->max_seq_len, m->padded_vocab, s));
                TRY(nc_launch_attention_shared(w.qh, kc, vc, kv->cache_seqlens, kv->shared_prefix, ly.window_left, w.y, B, H, Hkv,
                                               kv->max_seq_len, 0, w.shared_parts, w.shared_part_bytes, w.site(site), s));
                shared_done = true;
            }
        }
        if (shared_done) {
            // (q, the new cache rows and the attention output are already written)
        } else if (T == 1) {
            // decode: the attention workgroups finish their own q|k|v heads and append to the cache themselves
            const NcRopeSrc rope{qsrc.parts ? nullptr : w.qkv, qkv_w, qsrc, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin,
                                 m->rope_len, m->padded_vocab, nullptr, nullptr};
            TRY(nc_launch_attention_fused(rope, kc, vc, kv->cache_seqlens, ly.window_left, w.y, B, H, Hkv, kv->max_seq_len,
                                          w.attn_counters, w.attn_parts, w.attn_part_bytes, w.site(site), 0, 1, s));
        } else {
            if (qsrc.parts)
                TRY(nc_launch_qkv_rope_append_p(qsrc, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len,
                                                kv->cache_seqlens, kc, vc, w.qh, B, T, H, Hkv, kv->max_seq_len, m->padded_vocab, s));
            else
                TRY(nc_launch_qkv_rope_append(w.qkv, qkv_w, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len,
                                              kv->cache_seqlens, kc, vc, w.qh, B, T, H, Hkv, kv->max_seq_len, m->padded_vocab, s));
            TRY(nc_launch_attention(w.qh, kc, vc, kv->cache_seqlens, ly.window_left, w.y, B, T, H, Hkv, kv->max_seq_len, 0,
                                    w.attn_counters, w.attn_parts, w.attn_part_bytes, w.site(site), 0, 1, s));
        }
        if (tap_y) TRY(tap_copy(tap_y + (size_t)i * M * H * 128, w.y, (size_t)M * H * 128, s));
        TRY(lin.run(w.y, M, site, ly.w_attn_proj, ly.inv_attn_proj, one_seg(E), w.o, 0, 0.f, nullptr, E, H * 128, E, &pending_parts));
        pending_add = pending_parts.parts ? nullptr : w.o;
        site++;
        // x += attn_out; xn = norm(x)
        TRY(mix(nullptr, nullptr, nullptr, nullptr, nullptr, w.site(site)));
        // h2 = relu(c_fc(xn))^2 with its amax in the next slot
        TRY(lin.run(w.xn, M, site, ly.w_fc, ly.inv_fc, one_seg(4 * E), w.h2, 2, 0.f, w.site(site + 1), 4 * E, E, 4 * E, nullptr));
        site++;
        TRY(lin.run(w.h2, M, site, ly.w_mlp_proj, ly.inv_mlp_proj, one_seg(E), w.o, 0, 0.f, nullptr, E, 4 * E, E, &pending_parts));
        pending_add = pending_parts.parts ? nullptr : w.o;
        site++;
    }
    // x += mlp_out(last layer); x -= backout_lambda * x_backout; xn = norm(x)      (gpt.py:506-508)
    {
        const bool last_is_backout = (L - 1) == L / 2;     // L == 1 or 2
        if (last_is_backout) {
            // the saved rows and the subtraction need the same x1: do the add first, then the backout pass
            TRY(mix(nullptr, nullptr, nullptr, nullptr, w.xb, nullptr));
            pending_add = nullptr;
            pending_parts = NO_PARTIALS;
        }
        // every layer has read the positions by now: a one-token step may have them advanced here instead of by a launch of the caller's
        const bool bump = kv->advance != 0 && T == 1 && E % 8 == 0 && E <= 8192;
        NC_CHECK_ARG(kv->advance == 0 || bump, "gpt_forward: cache_desc.advance needs T == 1 (and n_embd %% 8 == 0, <= 8192)");
        TRY(mix(nullptr, nullptr, m->backout_lambda, w.xb, nullptr, w.site(site), bump ? (int32_t*)kv->cache_seqlens : nullptr, kv->advance));
        if (tap_x) TRY(tap_copy(tap_x + (size_t)L * M * E, w.xn, (size_t)M * E, s));
    }
    // lm_head.  Its activation scale is tensorwise over all M rows (that is what the reference quantizes),
    // even when only the last position of every row is projected.
    const bf16_t* head_in = w.xn;
    int head_rows = M;
    if (last_only && T > 1) {
        hipLaunchKernelGGL(gather_last_rows_kernel, dim3(B), dim3(256), 0, s, w.xn, w.xl, T, E);
        NC_CHECK_LAUNCH("gather_last_rows");
        head_in = w.xl;
        head_rows = B;
    }
    TRY(lin.run(head_in, head_rows, site, m->w_lm_head, m->inv_lm_head, one_seg(m->vocab_size), logits_out, 1, m->softcap, nullptr,
                m->vocab_size, E, m->vocab_size, nullptr));
    return 0;
}

extern "C" int nc_gpt_forward(const nc_model_desc* m, const nc_cache_desc* kv, const int64_t* idx, int B, int T, float* logits_out,
                              int last_only, void* workspace, size_t workspace_bytes, nc_stream_t stream) {
    return gpt_forward_impl(m, kv, idx, B, T, logits_out, last_only, workspace, workspace_bytes, nullptr, nullptr, (hipStream_t)stream);
}

extern "C" int nc_gpt_forward_tapped(const nc_model_desc* m, const nc_cache_desc* kv, const int64_t* idx, int B, int T, float* logits_out,
                                     int last_only, void* workspace, size_t workspace_bytes, uint16_t* tap_x, uint16_t* tap_y,
                                     nc_stream_t stream) {
    return gpt_forward_impl(m, kv, idx, B, T, logits_out, last_only, workspace, workspace_bytes, tap_x, tap_y, (hipStream_t)stream);
}
