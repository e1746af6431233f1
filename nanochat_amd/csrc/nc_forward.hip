// Host-side sequencing of one GPT.forward(idx, kv_cache=...) on a stream: the native replacement of the
// Python loop at nanochat/gpt.py:459-524 (and of the module calls it makes into gpt.py:84-153 and
// fp8.py:202-213).  One call enqueues every kernel of the step; no host synchronisation, no allocation.
//
// Workspace layout (carved from the caller's buffer, 256-byte aligned pieces), M = B*T rows:
//   x, x0, xn, xb, o      bf16 [M,E]        residual stream, its initial value, normed rows, backout, GEMM out
//   qkv                   bf16 [M,(H+2Hkv)*128]
//   qh, y                 bf16 [M,H*128]    rotated queries, attention output
//   h, h2                 bf16 [M,4E]       c_fc output, relu^2
//   a8                    u8   [M,4E]       quantized activations (input of the next GEMM)
//   xl                    bf16 [B,E]        last-position rows (last_only lm_head)
//   inv                   fp32 [4L+1]       activation inverse scales, one per FP8 linear input
//   amax                  u32  [4L+1]       amax slots, cleared once at the start of the call
//   attn                  fp32              split-K partials
#include <stdio.h>
#include "../../include/nanochat_amd.h"
#include "nc_common.h"
#include "nc_kernels.h"

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
    uint8_t* a8;
    float* inv;
    uint32_t* amax;
    void* attn;
    size_t attn_bytes;
    size_t total;
};

Workspace carve(const nc_model_desc* m, int B, int T, void* base) {
    const size_t M = (size_t)B * T, E = m->n_embd;
    const size_t qkv_w = (size_t)(m->n_head + 2 * m->n_kv_head) * 128;
    Carver c(base);
    Workspace w;
    w.x = c.take<bf16_t>(M * E);
    w.x0 = c.take<bf16_t>(M * E);
    w.xn = c.take<bf16_t>(M * E);
    w.xb = c.take<bf16_t>(M * E);
    w.o = c.take<bf16_t>(M * E);
    w.qkv = c.take<bf16_t>(M * qkv_w);
    w.qh = c.take<bf16_t>(M * m->n_head * 128);
    w.y = c.take<bf16_t>(M * m->n_head * 128);
    w.h = c.take<bf16_t>(M * 4 * E);
    w.h2 = c.take<bf16_t>(M * 4 * E);
    w.a8 = c.take<uint8_t>(M * 4 * E);
    w.xl = c.take<bf16_t>((size_t)B * E);
    w.inv = c.take<float>(4 * (size_t)m->n_layer + 1);
    w.amax = c.take<uint32_t>(4 * (size_t)m->n_layer + 1);
    w.attn_bytes = nc_attn_ws_bytes(B, T, m->n_head);
    w.attn = c.take<uint8_t>(w.attn_bytes);
    w.total = (c.off + 255) & ~(size_t)255;
    return w;
}

NcGemmSegs one_seg(int n) { return NcGemmSegs{1, {n, 0, 0, 0}}; }

__global__ void gather_last_rows_kernel(const bf16_t* __restrict__ x, bf16_t* __restrict__ out, int T, int E) {
    const int b = blockIdx.x;
    const bf16_t* src = x + ((size_t)b * T + (T - 1)) * E;
    for (int c = threadIdx.x; c < E; c += blockDim.x) out[(size_t)b * E + c] = src[c];
}
}  // namespace

extern "C" size_t nc_gpt_workspace_bytes(const nc_model_desc* model, int B, int T) {
    if (!model || B <= 0 || T <= 0) return 0;
    return carve(model, B, T, nullptr).total;
}

#define TRY(call)              \
    do {                       \
        int rc__ = (call);     \
        if (rc__) return rc__; \
    } while (0)

extern "C" int nc_gpt_forward(const nc_model_desc* m, const nc_cache_desc* kv, const int64_t* idx, int B, int T,
                              float* logits_out, int last_only, void* workspace, size_t workspace_bytes, nc_stream_t stream) {
    hipStream_t s = (hipStream_t)stream;
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
    int site = 0;   // index into inv / amax

    nc_clear_u32(w.amax, 4 * L + 1, s);
    TRY(nc_launch_embed_norm_smear(idx, m->wte, m->smear_w, m->smear_lambda, kv->prev_in, kv->prev_out, w.x, B, T, E,
                                   m->padded_vocab, s));
    // x0 is the post-smear embedding; layer 0 reads it through both x and x0 (gpt.py:495,500)
    if (hipMemcpyAsync(w.x0, w.x, (size_t)M * E * sizeof(bf16_t), hipMemcpyDeviceToDevice, s) != hipSuccess)
        NC_FAIL(-2, "gpt_forward: x0 copy failed");

    const bf16_t* pending_add = nullptr;   // GEMM output still to be added into the residual stream
    for (int i = 0; i < L; i++) {
        const nc_layer_desc& ly = m->layers[i];
        NC_CHECK_ARG(ly.w_qkv && ly.inv_qkv && ly.w_attn_proj && ly.w_fc && ly.w_mlp_proj, "gpt_forward: layer %d has no FP8 weights", i);
        // x += mlp_out(prev layer); [save backout]; x = rl*x + xl*x0; xn = norm(x)
        bf16_t* save = (i > 0 && (i - 1) == L / 2) ? w.xb : nullptr;
        TRY(nc_launch_mix_norm(w.x, pending_add, w.x0, m->resid_lambdas + i, m->x0_lambdas + i, nullptr, nullptr, save, w.xn, M, E,
                               w.amax + site, s));
        // q|k|v = FP8 linear(xn): one activation quantization, three weight scales
        TRY(nc_launch_convert_only(w.xn, (int64_t)M * E, w.a8, w.inv + site, w.amax + site, s));
        NcGemmSegs qkv_segs{3, {H * 128, (H + Hkv) * 128, qkv_w, 0}};
        TRY(nc_launch_gemm(w.a8, ly.w_qkv, w.inv + site, ly.inv_qkv, qkv_segs, w.qkv, 0, 0.f, M, qkv_w, E, qkv_w, 0, s));
        site++;
        bf16_t* kc = kv->k_cache + (size_t)i * layer_elems;
        bf16_t* vc = kv->v_cache + (size_t)i * layer_elems;
        TRY(nc_launch_qkv_rope_append(w.qkv, qkv_w, w.xn, E, idx, ly.ve_table, ly.ve_gate_w, m->cos, m->sin, m->rope_len,
                                      kv->cache_seqlens, kc, vc, w.qh, B, T, H, Hkv, kv->max_seq_len, m->padded_vocab, s));
        TRY(nc_launch_attention(w.qh, kc, vc, kv->cache_seqlens, ly.window_left, w.y, B, T, H, Hkv, kv->max_seq_len, 0, w.attn,
                                w.attn_bytes, w.amax + site, 0, s));
        // attention projection
        TRY(nc_launch_convert_only(w.y, (int64_t)M * H * 128, w.a8, w.inv + site, w.amax + site, s));
        TRY(nc_launch_gemm(w.a8, ly.w_attn_proj, w.inv + site, ly.inv_attn_proj, one_seg(E), w.o, 0, 0.f, M, E, H * 128, E, 0, s));
        site++;
        // x += attn_out; xn = norm(x)
        TRY(nc_launch_mix_norm(w.x, w.o, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, w.xn, M, E, w.amax + site, s));
        TRY(nc_launch_convert_only(w.xn, (int64_t)M * E, w.a8, w.inv + site, w.amax + site, s));
        TRY(nc_launch_gemm(w.a8, ly.w_fc, w.inv + site, ly.inv_fc, one_seg(4 * E), w.h, 0, 0.f, M, 4 * E, E, 4 * E, 0, s));
        site++;
        TRY(nc_launch_relu2(w.h, w.h2, (int64_t)M * 4 * E, w.amax + site, s));
        TRY(nc_launch_convert_only(w.h2, (int64_t)M * 4 * E, w.a8, w.inv + site, w.amax + site, s));
        TRY(nc_launch_gemm(w.a8, ly.w_mlp_proj, w.inv + site, ly.inv_mlp_proj, one_seg(E), w.o, 0, 0.f, M, E, 4 * E, E, 0, s));
        site++;
        pending_add = w.o;
    }
    // x += mlp_out(last layer); x -= backout_lambda * x_backout; xn = norm(x)      (gpt.py:506-508)
    {
        const bool last_is_backout = (L - 1) == L / 2;     // only when L == 1
        bf16_t* save = last_is_backout ? w.xb : nullptr;
        if (last_is_backout) {
            // the saved rows and the subtraction need the same x1: do the add first, then the backout pass
            TRY(nc_launch_mix_norm(w.x, pending_add, nullptr, nullptr, nullptr, nullptr, nullptr, save, w.xn, M, E, nullptr, s));
            pending_add = nullptr;
        }
        TRY(nc_launch_mix_norm(w.x, pending_add, nullptr, nullptr, nullptr, m->backout_lambda, w.xb, nullptr, w.xn, M, E,
                               w.amax + site, s));
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
    TRY(nc_launch_convert_only(head_in, (int64_t)head_rows * E, w.a8, w.inv + site, w.amax + site, s));
    NcGemmSegs head_seg{1, {m->vocab_size, 0, 0, 0}};
    TRY(nc_launch_gemm(w.a8, m->w_lm_head, w.inv + site, m->inv_lm_head, head_seg, logits_out, 1, m->softcap, head_rows,
                       m->vocab_size, E, m->vocab_size, 0, s));
    return 0;
}
