// extern "C" surface of libnanochat_amd.so: argument validation, the thread-local error message and
// thin forwarding into the launch functions.  Declarations and reference citations: include/nanochat_amd.h.
#include <stdarg.h>
#include <stdio.h>
#include "../../include/nanochat_amd.h"
#include "nc_common.h"
#include "nc_kernels.h"
#include "nc_rope.h"

static thread_local char g_error[512] = "";

void nc_set_error(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
}

extern "C" {

int nc_abi_version(void) { return 2; }
const char* nc_last_error(void) { return g_error; }

int nc_fp8_quantize_tensorwise(const void* x, int x_dtype, int64_t n, uint8_t* out, float* scale_out, float* inv_scale_out,
                               uint32_t* amax_ws, int encoder, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "fp8_quantize: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_quantize(x, x_dtype, n, 0, out, scale_out, inv_scale_out, amax_ws, encoder, (hipStream_t)stream);
}

int nc_fp8_quantize_tensorwise_as(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                  float* inv_scale_out, uint32_t* amax_ws, int encoder, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "fp8_quantize: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_quantize(x, x_dtype, n, fp8_format, out, scale_out, inv_scale_out, amax_ws, encoder, (hipStream_t)stream);
}

size_t nc_fp8_quantize_state_bytes(void) { return NC_QUANTIZE_STATE_BYTES; }

int nc_fp8_quantize_tensorwise_fused(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                     float* inv_scale_out, void* state, int encoder, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "fp8_quantize: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_quantize_fused(x, x_dtype, n, fp8_format, out, scale_out, inv_scale_out, (uint32_t*)state, encoder, (hipStream_t)stream);
}

int nc_fp8_quantize_tensorwise_fused_bounded(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                             float* inv_scale_out, void* state, int encoder, uint32_t spin_limit, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "fp8_quantize: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_quantize_fused(x, x_dtype, n, fp8_format, out, scale_out, inv_scale_out, (uint32_t*)state, encoder, (hipStream_t)stream,
                                    spin_limit);
}

int nc_fp8_encode_with_scale(const uint16_t* x, int64_t n, float scale, int fp8_format, uint8_t* out, int encoder, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "fp8_encode: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_encode_with_scale(x, n, scale, fp8_format, out, encoder, (hipStream_t)stream);
}

int nc_fp8_quantize_tensorwise_transposed(const uint16_t* x, int rows, int cols, int fp8_format, uint8_t* out, uint8_t* out_t, float* scale_out,
                                          float* inv_scale_out, uint32_t* amax_ws, nc_stream_t stream) {
    return nc_launch_quantize_transposed(x, rows, cols, fp8_format, out, out_t, scale_out, inv_scale_out, amax_ws, (hipStream_t)stream);
}

int nc_fp8_transpose(const uint8_t* src, int rows, int cols, uint8_t* dst, nc_stream_t stream) {
    return nc_launch_transpose_u8(src, rows, cols, dst, (hipStream_t)stream);
}

int nc_e4m3_encode_with_scale(const uint16_t* x, int64_t n, float scale, uint8_t* out, int encoder, nc_stream_t stream) {
    NC_CHECK_ARG(encoder == 0 || encoder == 1, "e4m3_encode: encoder must be 0 (hardware) or 1 (software)");
    return nc_launch_encode_with_scale(x, n, scale, 0, out, encoder, (hipStream_t)stream);
}

static int segs_from(const int32_t* seg_ends, int nseg, int N, NcGemmSegs* segs) {
    *segs = NcGemmSegs{1, {N, 0, 0, 0}};
    if (seg_ends) {
        NC_CHECK_ARG(nseg >= 1 && nseg <= 4, "fp8_gemm: 1..4 column segments supported, got %d", nseg);
        segs->nseg = nseg;
        for (int i = 0; i < nseg; i++) segs->end[i] = seg_ends[i];
    }
    return 0;
}

int nc_fp8_gemm_tn(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, const int32_t* seg_ends, int nseg,
                   void* out, int out_kind, float softcap, int M, int N, int K, int ldc, int kernel, void* workspace,
                   size_t workspace_bytes, nc_stream_t stream) {
    NcGemmSegs segs;
    if (int rc = segs_from(seg_ends, nseg, N, &segs)) return rc;
    return nc_launch_gemm(a, b, inv_a, inv_b, segs, out, out_kind, softcap, M, N, K, ldc, kernel, workspace, workspace_bytes,
                          (hipStream_t)stream);
}

int nc_fp8_gemm_tn_grad(const uint8_t* a_e5m2, const uint8_t* b, const float* inv_a, const float* inv_b, void* out, int M, int N, int K,
                        int ldc, int kernel, nc_stream_t stream) {
    NcGemmSegs segs{1, {N, 0, 0, 0}};
    return nc_launch_gemm(a_e5m2, b, inv_a, inv_b, segs, out, 0, 0.f, M, N, K, ldc, kernel, nullptr, 0, (hipStream_t)stream, 1);
}

int nc_fp8_gemm_tn_relu2(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, void* out, uint32_t* out_amax, int M,
                         int N, int K, int ldc, int kernel, nc_stream_t stream) {
    NcGemmSegs segs{1, {N, 0, 0, 0}};
    return nc_launch_gemm(a, b, inv_a, inv_b, segs, out, 2, 0.f, M, N, K, ldc, kernel, nullptr, 0, (hipStream_t)stream, 0, out_amax);
}

size_t nc_fp8_small_m_workspace_bytes(int M, int N, int K) {
    if (M < 1 || M > 128 || N < 1 || K < 1) return 0;
    return nc_gemm_decode_partial_bytes(M, N, K);
}

int nc_fp8_linear_small_m(const uint16_t* a_bf16, const uint32_t* a_amax, const uint8_t* b, const float* inv_b,
                          const int32_t* seg_ends, int nseg, void* out, int out_kind, float softcap, uint32_t* out_amax, int M, int N,
                          int K, int ldc, void* workspace, size_t workspace_bytes, int ksplits, nc_stream_t stream) {
    NcGemmSegs segs;
    if (int rc = segs_from(seg_ends, nseg, N, &segs)) return rc;
    NC_CHECK_ARG(out && inv_b, "fp8_linear_small_m: null pointer");
    hipStream_t s = (hipStream_t)stream;
    // left to choose (ksplits <= 0), the launch picks the form; without room for the partial sums it would need, one split
    int ks = ksplits > 0 ? ksplits : 0;
    if (ksplits <= 0) {
        const int want = nc_gemm_decode_splits(N, K);
        if (want > 1 && (!workspace || workspace_bytes < (size_t)want * M * N * sizeof(float))) ks = 1;
    }
    int used = 1;
    if (int rc = nc_launch_gemm_decode(a_bf16, 1, a_amax, nullptr, b, inv_b, segs, out, out_kind, softcap, out_amax, M, N, K, ldc,
                                       (float*)workspace, workspace_bytes, ks, &used, s))
        return rc;
    if (used > 1)
        return nc_launch_finish_partials((const float*)workspace, used, a_amax, nullptr, inv_b, segs, out, out_kind, softcap, out_amax, M,
                                         N, ldc, s);
    return 0;
}

int nc_rmsnorm(const uint16_t* x, uint16_t* out, int rows, int cols, uint32_t* amax_ws, nc_stream_t stream) {
    return nc_launch_rmsnorm(x, out, rows, cols, amax_ws, (hipStream_t)stream);
}

int nc_embed_norm_smear(const int64_t* idx, const uint16_t* wte, const float* smear_w, const float* smear_lambda,
                        const uint16_t* prev_in, uint16_t* prev_out, uint16_t* x_out, int B, int T, int E, int vocab_rows,
                        nc_stream_t stream) {
    return nc_launch_embed_norm_smear(idx, wte, smear_w, smear_lambda, prev_in, prev_out, x_out, nullptr, B, T, E, vocab_rows, nullptr, 0,
                                      (hipStream_t)stream);
}

int nc_mix_norm(uint16_t* x, const uint16_t* add, const uint16_t* x0, const float* resid_lambda, const float* x0_lambda,
                const float* backout_lambda, const uint16_t* backout_src, uint16_t* backout_save, uint16_t* xn_out, int rows,
                int cols, uint32_t* amax_ws, nc_stream_t stream) {
    return nc_launch_mix_norm(x, add, x0, resid_lambda, x0_lambda, backout_lambda, backout_src, backout_save, xn_out, rows, cols,
                              amax_ws, (hipStream_t)stream);
}

int nc_relu2(const uint16_t* h, uint16_t* out, int64_t n, uint32_t* amax_ws, nc_stream_t stream) {
    return nc_launch_relu2(h, out, n, amax_ws, (hipStream_t)stream);
}

int nc_qkv_rope_append(const uint16_t* qkv, int ld_qkv, const uint16_t* xn, int ld_xn, const int64_t* idx, const uint16_t* ve_table,
                       const float* ve_gate_w, const uint16_t* cos, const uint16_t* sin, int rope_len, const int32_t* cache_seqlens,
                       uint16_t* k_cache, uint16_t* v_cache, uint16_t* q_out, int B, int T, int H, int Hkv, int Tmax, int vocab_rows,
                       nc_stream_t stream) {
    return nc_launch_qkv_rope_append(qkv, ld_qkv, xn, ld_xn, idx, ve_table, ve_gate_w, cos, sin, rope_len, cache_seqlens, k_cache,
                                     v_cache, q_out, B, T, H, Hkv, Tmax, vocab_rows, (hipStream_t)stream);
}

size_t nc_attention_workspace_bytes(int B, int T, int H, int Tmax) {
    (void)Tmax;
    if (B <= 0 || T <= 0 || H <= 0) return 0;
    return nc_attn_counter_bytes(B, T, H) + nc_attn_partial_bytes(B, T, H);
}

int nc_decode_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int32_t* cache_seqlens,
                        int window_left, uint16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                        void* workspace, size_t workspace_bytes, uint32_t* amax_ws, int splits, nc_stream_t stream) {
    const size_t cb = nc_attn_counter_bytes(B > 0 ? B : 1, T > 0 ? T : 1, H > 0 ? H : 1);
    uint32_t* counters = (workspace && workspace_bytes > cb) ? (uint32_t*)workspace : nullptr;
    void* parts = counters ? (uint8_t*)workspace + cb : nullptr;
    return nc_launch_attention(q, k_cache, v_cache, cache_seqlens, window_left, out, B, T, H, Hkv, Tmax, seqlens_include_new,
                               counters, parts, counters ? workspace_bytes - cb : 0, amax_ws, splits, 0, (hipStream_t)stream);
}

size_t nc_decode_attention_shared_workspace_bytes(int B, int H, int Hkv, int shared_len) {
    if (B <= 0 || H <= 0 || Hkv <= 0 || shared_len <= 0 || H % Hkv != 0) return 0;
    return nc_attn_shared_partial_bytes(B, H, Hkv, shared_len);
}

int nc_decode_attention_shared(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int32_t* cache_seqlens,
                               int shared_len, int window_left, uint16_t* out, int B, int H, int Hkv, int Tmax, int seqlens_include_new,
                               void* workspace, size_t workspace_bytes, uint32_t* amax_ws, nc_stream_t stream) {
    NC_CHECK_ARG(q && k_cache && v_cache && cache_seqlens && out && workspace, "decode_attention_shared: null pointer");
    return nc_launch_attention_shared(q, k_cache, v_cache, cache_seqlens, shared_len, window_left, out, B, H, Hkv, Tmax, seqlens_include_new,
                                      workspace, workspace_bytes, amax_ws, (hipStream_t)stream);
}

static void split_attention_workspace(void* workspace, size_t workspace_bytes, int B, int T, int H, uint32_t** counters, void** parts,
                                      size_t* part_bytes) {
    const size_t cb = nc_attn_counter_bytes(B > 0 ? B : 1, T > 0 ? T : 1, H > 0 ? H : 1);
    *counters = (workspace && workspace_bytes > cb) ? (uint32_t*)workspace : nullptr;
    *parts = *counters ? (uint8_t*)workspace + cb : nullptr;
    *part_bytes = *counters ? workspace_bytes - cb : 0;
}

int nc_decode_attention_append(const uint16_t* q, const uint16_t* k_new, const uint16_t* v_new, uint16_t* k_cache, uint16_t* v_cache,
                               const int32_t* cache_seqlens, int window_left, uint16_t* out, int B, int T, int H, int Hkv, int Tmax,
                               void* workspace, size_t workspace_bytes, uint32_t* amax_ws, int splits, nc_stream_t stream) {
    uint32_t* counters;
    void* parts;
    size_t part_bytes;
    split_attention_workspace(workspace, workspace_bytes, B, T, H, &counters, &parts, &part_bytes);
    return nc_launch_attention_append(q, k_new, v_new, k_cache, v_cache, cache_seqlens, window_left, out, B, T, H, Hkv, Tmax, counters, parts,
                                      part_bytes, amax_ws, splits, (hipStream_t)stream);
}

int nc_qkv_rope_append_attention(const uint16_t* qkv, int ld_qkv, const uint16_t* xn, int ld_xn, const int64_t* idx,
                                 const uint16_t* ve_table, const float* ve_gate_w, const uint16_t* cos, const uint16_t* sin, int rope_len,
                                 const int32_t* cache_seqlens, uint16_t* k_cache, uint16_t* v_cache, int window_left, uint16_t* out, int B,
                                 int H, int Hkv, int Tmax, int vocab_rows, void* workspace, size_t workspace_bytes, uint32_t* amax_ws,
                                 int splits, nc_stream_t stream) {
    NC_CHECK_ARG(qkv && ld_qkv >= (H + 2 * Hkv) * 128, "qkv_rope_append_attention: qkv rows of %d elements needed", (H + 2 * Hkv) * 128);
    uint32_t* counters;
    void* parts;
    size_t part_bytes;
    split_attention_workspace(workspace, workspace_bytes, B, 1, H, &counters, &parts, &part_bytes);
    NcRopeSrc rope{qkv, ld_qkv, NcPartialSrc{nullptr, 0, 0, 0, nullptr, nullptr, 0, 0}, xn, ld_xn, idx, ve_table, ve_gate_w, cos, sin,
                   rope_len, vocab_rows, nullptr, nullptr};
    return nc_launch_attention_fused(rope, k_cache, v_cache, cache_seqlens, window_left, out, B, H, Hkv, Tmax, counters, parts, part_bytes,
                                     amax_ws, splits, 0, (hipStream_t)stream);
}

size_t nc_decode_attention_static_max_row_heads(void) { return nc_attention_static_max_row_heads(); }

int nc_decode_attention_static(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int32_t* cache_seqlens,
                               int window_left, uint16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                               uint32_t* amax_ws, int splits, nc_stream_t stream) {
    return nc_launch_attention_static(q, k_cache, v_cache, cache_seqlens, window_left, out, B, T, H, Hkv, Tmax, seqlens_include_new, amax_ws,
                                      splits, (hipStream_t)stream);
}

int nc_decode_attention_plan(int B, int T, int Hkv, int window_left, int Tmax, int splits, int* splits_out, int* heads_per_workgroup_out) {
    NC_CHECK_ARG(B > 0 && T > 0 && Hkv > 0 && Tmax > 0, "decode_attention_plan: bad shape");
    nc_attention_plan(B, T, Hkv, window_left, Tmax, splits, splits_out, heads_per_workgroup_out);
    return 0;
}

int nc_softcap(const uint16_t* raw, float* out, int64_t n, float softcap, nc_stream_t stream) {
    return nc_launch_softcap(raw, out, n, softcap, (hipStream_t)stream);
}

int nc_kv_cache_prefill(const void* src, void* dst, int layers, int src_rows, int dst_rows, int src_tmax, int dst_tmax, int n_tokens,
                        int token_bytes, nc_stream_t stream) {
    return nc_launch_kv_prefill_copy(src, dst, layers, src_rows, dst_rows, src_tmax, dst_tmax, n_tokens, token_bytes, (hipStream_t)stream);
}

int nc_sample(const float* logits, int B, int V, int ld, float temperature, int top_k, const float* noise, int64_t* out_ids,
              nc_stream_t stream) {
    return nc_launch_sample(logits, B, V, ld, temperature, top_k, noise, out_ids, (hipStream_t)stream);
}

}  // extern "C"
