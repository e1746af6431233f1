/* nanochat_amd -- C ABI of the MI355X (gfx950) FP8 + KV-cache decode path.
 *
 * Every entry point replaces one piece of the reference's hot path (citations are into the
 * reference tree).  Conventions:
 *   - all pointers are DEVICE pointers unless a parameter says "host";
 *   - work is enqueued on `stream` (a hipStream_t passed as void*); nothing synchronises;
 *   - nothing allocates or frees device memory: callers own inputs, outputs and workspaces;
 *   - return 0 on success, negative on error; nc_last_error() gives the message of the last
 *     failure on the calling thread (the Python host re-raises it as AssertionError/ValueError,
 *     which is how the reference reports the same conditions);
 *   - bf16 tensors are raw uint16_t bit patterns, e4m3 tensors raw uint8_t (OCP e4m3fn, the
 *     encoding of torch.float8_e4m3fn);
 *   - re-entrancy: every entry point may be called from any thread on any stream, and keeps no state between
 *     calls beyond per-process caches of device facts (CU count, LDS attributes, occupancy), with TWO
 *     exceptions, both process-wide and not thread-safe: the measurement aid (nc_profile_*: one set of event
 *     pairs and counters per process, to be switched on by one thread while no other thread launches), and
 *     nc_decode_attention_static (one scratch array per GPU shared by all its calls: calls on one GPU must not
 *     overlap in time, whatever stream or thread they come from).  A caller-provided state or workspace block
 *     (quantizer state, split workspaces, the forward's workspace) serves one call at a time: calls that may
 *     overlap need a block each.
 */
#ifndef NANOCHAT_AMD_H
#define NANOCHAT_AMD_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* nc_stream_t;

int nc_abi_version(void);
const char* nc_last_error(void);

/* (1) Tensorwise dynamic quantization: nanochat/fp8.py:81-107 (_to_fp8).
 * x_dtype: 0 = bf16, 1 = fp32.  Writes n payload bytes, *inv_scale_out (= 1/scale, what
 * torch._scaled_mm takes) and, if not NULL, *scale_out.  amax_ws: one uint32 of scratch that
 * the call clears itself.  encoder: 0 = hardware convert, 1 = integer software encoder. */
int nc_fp8_quantize_tensorwise(const void* x, int x_dtype, int64_t n, uint8_t* out, float* scale_out,
                               float* inv_scale_out, uint32_t* amax_ws, int encoder, nc_stream_t stream);

/* Encoder only, with a caller-given scale (no amax pass); x is bf16.  For exhaustive checks of
 * the cast at nanochat/fp8.py:101-103. */
int nc_e4m3_encode_with_scale(const uint16_t* x, int64_t n, float scale, uint8_t* out, int encoder,
                              nc_stream_t stream);

/* The same with the fp8 format as a parameter: fp8_format 0 = e4m3fn (activations, weights), 1 = e5m2 (OCP, the
 * encoding of torch.float8_e5m2; saturates at 57344), which nanochat/fp8.py:165 uses for the output gradient. */
int nc_fp8_quantize_tensorwise_as(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                  float* inv_scale_out, uint32_t* amax_ws, int encoder, nc_stream_t stream);
int nc_fp8_encode_with_scale(const uint16_t* x, int64_t n, float scale, int fp8_format, uint8_t* out, int encoder,
                             nc_stream_t stream);

/* The same quantization in ONE launch where the tensor allows it (bf16 input, n a multiple of 16, up to roughly 30 million
 * elements: what the registers of the workgroups resident on the chip hold): every element is read from memory once, the
 * workgroups meet on the tensor's amax, the payload is converted from registers.  Other tensors take the two passes of
 * nc_fp8_quantize_tensorwise_as; results are bit-identical either way.  state: nc_fp8_quantize_state_bytes() bytes, 128-byte
 * aligned, ALL ZERO before the first call with it; every call leaves it all zero (words 257 and 320 excepted, see below),
 * so one allocation serves all calls that do not overlap in time; calls that overlap need a state each.  The one-launch grid
 * is sized to half of what the GPU holds of it, so that two such grids at once (of this or any other process on the GPU) are
 * both resident; with more of them at once a workgroup can wait for peers that have no slot yet.  That wait is bounded: a
 * workgroup whose wait runs out works the amax out by itself from the whole tensor (slow, same bits) and is counted in word
 * 257 of the state, which no kernel reads or clears -- a host that wants to know reads it; the results are correct either way.
 * Word 320 is scratch of the two-pass path. */
size_t nc_fp8_quantize_state_bytes(void);
int nc_fp8_quantize_tensorwise_fused(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                     float* inv_scale_out, void* state, int encoder, nc_stream_t stream);
/* The same with the bound of the wait given by the caller: spin_limit polls of a few hundred nanoseconds each (the entry above
 * uses about four million).  0 makes nearly every workgroup take the slow way at once, which is how that way is tested. */
int nc_fp8_quantize_tensorwise_fused_bounded(const void* x, int x_dtype, int64_t n, int fp8_format, uint8_t* out, float* scale_out,
                                             float* inv_scale_out, void* state, int encoder, uint32_t spin_limit, nc_stream_t stream);

/* Tensorwise quantization of a bf16 matrix x[rows][cols] that writes the payload twice from one read of x: out[rows][cols] and
 * out_t[cols][rows].  The backward GEMMs of nanochat/fp8.py:156-192 take the output gradient both ways (grad_output in e5m2 for
 * grad_input, fp8.py:166-177; its transpose for grad_weight, fp8.py:179-190) and the saved input transposed (_to_col_major,
 * fp8.py:110-118,181-182): the separate transposes of those payloads drop out.  Scale, inverse scale and payload bits are those of
 * nc_fp8_quantize_tensorwise_as.  rows and cols multiples of 16, pointers 16-byte aligned; amax_ws: one uint32, cleared by the call. */
int nc_fp8_quantize_tensorwise_transposed(const uint16_t* x, int rows, int cols, int fp8_format, uint8_t* out, uint8_t* out_t,
                                          float* scale_out, float* inv_scale_out, uint32_t* amax_ws, nc_stream_t stream);

/* dst[cols][rows] = transpose of the fp8 payload src[rows][cols]: the memory rearrangement of _to_col_major and
 * .t().contiguous() at nanochat/fp8.py:110-118,169,181-182 (the backward GEMMs want the summed index contiguous in
 * both operands).  rows and cols multiples of 16, pointers 16-byte aligned. */
int nc_fp8_transpose(const uint8_t* src, int rows, int cols, uint8_t* dst, nc_stream_t stream);

/* (2) FP8 scaled GEMM: torch._scaled_mm as called at nanochat/fp8.py:143-153.
 * out[M,N] = bf16((a[M,K] . b[N,K]^T, fp32 accumulate) * *inv_a * inv_b[seg(n)]).
 * b may stack up to 4 weight matrices along N; seg_ends (HOST array of nseg exclusive column ends)
 * says where each one stops and inv_b holds one inverse scale per segment.
 * out_kind 0: bf16 out with leading dimension ldc.  out_kind 1: fp32 out of
 * softcap*tanh(bf16(v)/softcap), i.e. lm_head followed by nanochat/gpt.py:512-515.
 * kernel: 0 auto, 1 small-M (M<=128), 4 plain-load tile 128x128 (any operand size), 5/6/7 buffer-load tiles
 * 128x128 / 256x128 / 256x256 (operands below 2 GiB each), 8 direct-to-LDS 256x256 tiles and 9 their persistent
 * form (bf16 output, K a multiple of 128; 9 also needs ceil(M/256) in {8,16,...,256}), 10 / 11 buffer-load tiles 64x128 / 96x128,
 * 12..15 direct-to-LDS tiles of 256 x 128 / 160 / 192 / 224 (one tile per workgroup), 16 / 17 / 18 direct-to-LDS tiles of 64 / 96 / 128 x 128
 * through four LDS stages (12..18: bf16 output, K a multiple of 128).
 * workspace (may be NULL): lets the small-M kernel split K over workgroups (fp32 partial sums, added
 * in a fixed order by a finishing kernel); size from nc_fp8_small_m_workspace_bytes(), 16-byte aligned. */
int nc_fp8_gemm_tn(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b,
                   const int32_t* seg_ends, int nseg, void* out, int out_kind, float softcap, int M, int N,
                   int K, int ldc, int kernel, void* workspace, size_t workspace_bytes, nc_stream_t stream);

/* The backward GEMMs of nanochat/fp8.py:166-190 (torch._scaled_mm with an e5m2 first operand):
 * out[M,N] = bf16((a[M,K] . b[N,K]^T, fp32 accumulate) * *inv_a * *inv_b), a in e5m2 (the quantized output gradient or
 * its transpose), b in e4m3fn (the transposed weight or input payload saved by the forward), K contiguous in both.
 *   grad_input [B,K']  = nc_fp8_gemm_tn_grad(go[B,N'],   wT[K',N'], ...)   M=B,  N=K', K=N'
 *   grad_weight[N',K'] = nc_fp8_gemm_tn_grad(goT[N',B],  xT[K',B],  ...)   M=N', N=K', K=B
 * kernel: 0 auto, 5 (128x128 tiles, any K multiple of 16), 8 / 9 (direct-to-LDS 256x256 tiles, K multiple of 128), 12..15 (direct-to-LDS
 * tiles of 256 x 128 / 160 / 192 / 224, K multiple of 128). */
int nc_fp8_gemm_tn_grad(const uint8_t* a_e5m2, const uint8_t* b, const float* inv_a, const float* inv_b, void* out, int M,
                        int N, int K, int ldc, int kernel, nc_stream_t stream);

/* The MLP's first linear with its activation (nanochat/gpt.py:138-139, c_fc then relu().square()) for M > 128 rows:
 * out[M,N] = bf16(relu(bf16(v))^2), v as in nc_fp8_gemm_tn, and atomicMax(*out_amax, fp32 bits of max(out)) so that the
 * next tensorwise quantization needs no amax pass; the caller clears *out_amax.  kernel: 0 auto, 5..9, 12..18. */
int nc_fp8_gemm_tn_relu2(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, void* out,
                         uint32_t* out_amax, int M, int N, int K, int ldc, int kernel, nc_stream_t stream);

/* (1)+(2) fused for decode, M <= 128: Float8Linear.forward (nanochat/fp8.py:202-213) in one launch.
 * a_bf16 [M,K] is quantized inside the kernel with the tensorwise scale derived from *a_amax (fp32
 * bits of max|a|, e.g. produced by nc_rmsnorm / nc_mix_norm / nc_decode_attention), bit-identical to
 * nc_fp8_quantize_tensorwise followed by nc_fp8_gemm_tn.  out_kind 0/1 as above; out_kind 2 writes
 * bf16 relu(bf16(v))^2 (nanochat/gpt.py:139) and max-reduces it into *out_amax.  ksplits 0 = choose. */
size_t nc_fp8_small_m_workspace_bytes(int M, int N, int K);
int nc_fp8_linear_small_m(const uint16_t* a_bf16, const uint32_t* a_amax, const uint8_t* b, const float* inv_b,
                          const int32_t* seg_ends, int nseg, void* out, int out_kind, float softcap,
                          uint32_t* out_amax, int M, int N, int K, int ldc, void* workspace, size_t workspace_bytes,
                          int ksplits, nc_stream_t stream);

/* (4a) Parameter-free RMSNorm over the last dimension: nanochat/gpt.py:42-43.  If amax_ws is not
 * NULL the kernel also atomically max-reduces |out| into it (fp32 bits; caller clears it). */
int nc_rmsnorm(const uint16_t* x, uint16_t* out, int rows, int cols, uint32_t* amax_ws, nc_stream_t stream);

/* (4b) Embedding gather + norm + smear: nanochat/gpt.py:471-492.  idx [B,T] int64; wte bf16
 * [vocab_rows,E]; smear_w fp32 [24]; smear_lambda fp32 [1]; prev_in bf16 [B,E] or NULL (the
 * KVCache.prev_embedding of the previous call); prev_out bf16 [B,E]; x_out bf16 [B*T,E]. */
int nc_embed_norm_smear(const int64_t* idx, const uint16_t* wte, const float* smear_w, const float* smear_lambda,
                        const uint16_t* prev_in, uint16_t* prev_out, uint16_t* x_out, int B, int T, int E,
                        int vocab_rows, nc_stream_t stream);

/* (4c) Residual add, per-layer lambda mix or backout, RMSNorm: nanochat/gpt.py:500, 151-152, 503-508.
 *   x1 = x (+ add);  backout_save <- x1 (if not NULL);
 *   x2 = rl*x1 + xl*x0 (if resid_lambda)  |  x1 - bl*backout_src (if backout_lambda)  |  x1;
 *   x <- x2 (in place);  xn_out <- rms_norm(x2);  amax_ws <- max|xn_out| (if not NULL). */
int nc_mix_norm(uint16_t* x, const uint16_t* add, const uint16_t* x0, const float* resid_lambda,
                const float* x0_lambda, const float* backout_lambda, const uint16_t* backout_src,
                uint16_t* backout_save, uint16_t* xn_out, int rows, int cols, uint32_t* amax_ws,
                nc_stream_t stream);

/* relu(h)^2 elementwise in bf16 (+ amax): nanochat/gpt.py:139. */
int nc_relu2(const uint16_t* h, uint16_t* out, int64_t n, uint32_t* amax_ws, nc_stream_t stream);

/* (4d) Rotary + QK-norm + 1.2 gain on q and k, value-embedding gate on v, and the in-place KV-cache
 * append: nanochat/gpt.py:89-104 and nanochat/flash_attention.py:167-170.  head_dim is 128.
 * qkv bf16 [B*T, ld_qkv] = q heads | k heads | v heads; xn bf16 [B*T, ld_xn] (gate input, first 12
 * channels); ve_table bf16 [vocab_rows, Hkv*128] or NULL; ve_gate_w fp32 [Hkv,12]; cos/sin bf16
 * [rope_len,64]; cache_seqlens int32 [B] = tokens in the cache BEFORE this call; k_cache/v_cache
 * bf16 [B,Tmax,Hkv,128] of this layer; q_out bf16 [B*T,H,128].  Token t of row b goes to slot
 * cache_seqlens[b]+t; slots outside [0,Tmax) are skipped. */
int nc_qkv_rope_append(const uint16_t* qkv, int ld_qkv, const uint16_t* xn, int ld_xn, const int64_t* idx,
                       const uint16_t* ve_table, const float* ve_gate_w, const uint16_t* cos, const uint16_t* sin,
                       int rope_len, const int32_t* cache_seqlens, uint16_t* k_cache, uint16_t* v_cache,
                       uint16_t* q_out, int B, int T, int H, int Hkv, int Tmax, int vocab_rows, nc_stream_t stream);

/* (3) Attention of T new tokens per row over the KV cache (decode: T = 1): flash_attn_with_kvcache
 * as called at nanochat/gpt.py:113-120 (nanochat/flash_attention.py:139-185), after the append.
 * q bf16 [B*T,H,128]; caches bf16 [B,Tmax,Hkv,128]; out bf16 [B*T,H,128].
 * Query t of row b sees keys [max(0,p-window_left), p], p = cache_seqlens[b] + t (window_left < 0:
 * unlimited).  seqlens_include_new: set to 1 if cache_seqlens was already advanced by T.
 * splits: 0 = choose; workspace must hold nc_attention_workspace_bytes() when more than one split
 * is used.  amax_ws as above (or NULL). */
size_t nc_attention_workspace_bytes(int B, int T, int H, int Tmax);
int nc_decode_attention(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                        const int32_t* cache_seqlens, int window_left, uint16_t* out, int B, int T, int H, int Hkv,
                        int Tmax, int seqlens_include_new, void* workspace, size_t workspace_bytes,
                        uint32_t* amax_ws, int splits, nc_stream_t stream);

/* The same call with the new keys and values handed over, as the reference hands them: flash_attn_with_kvcache(q, k_cache,
 * v_cache, k=k_new, v=v_new, cache_seqlens=..., causal=True, window_size=(w, 0)) at nanochat/gpt.py:113-120, whose in-place
 * insert is nanochat/flash_attention.py:167-170.  k_new, v_new bf16 [B*T,Hkv,128] go to slots cache_seqlens[b] .. +T-1 of the
 * caches (slots outside [0,Tmax) are skipped), then the T queries of every row attend as above; cache_seqlens counts the
 * tokens BEFORE this call and is not advanced (the caller does that, nanochat/gpt.py:122-123).  With T = 1 the attention
 * workgroups append their own heads and take the new key and value from on-chip memory. */
int nc_decode_attention_append(const uint16_t* q, const uint16_t* k_new, const uint16_t* v_new, uint16_t* k_cache,
                               uint16_t* v_cache, const int32_t* cache_seqlens, int window_left, uint16_t* out, int B, int T,
                               int H, int Hkv, int Tmax, void* workspace, size_t workspace_bytes, uint32_t* amax_ws, int splits,
                               nc_stream_t stream);

/* (4d)+(3) in one launch for decode (one new token per row): nc_qkv_rope_append followed by nc_decode_attention, i.e.
 * nanochat/gpt.py:89-120 from the q|k|v linear's output to the attention output: rotary, QK-norm and gain on q and k, the
 * value-embedding gate on v, the in-place append at cache_seqlens[b], attention over [max(0,p-window_left), p].  Arguments
 * as for the two calls; out bf16 [B,H,128].  This is the kernel the whole-model forward uses at decode. */
int nc_qkv_rope_append_attention(const uint16_t* qkv, int ld_qkv, const uint16_t* xn, int ld_xn, const int64_t* idx,
                                 const uint16_t* ve_table, const float* ve_gate_w, const uint16_t* cos, const uint16_t* sin,
                                 int rope_len, const int32_t* cache_seqlens, uint16_t* k_cache, uint16_t* v_cache,
                                 int window_left, uint16_t* out, int B, int H, int Hkv, int Tmax, int vocab_rows,
                                 void* workspace, size_t workspace_bytes, uint32_t* amax_ws, int splits, nc_stream_t stream);

/* nc_decode_attention (one new token per row, already appended) for a batch whose rows all begin with the same shared_len cached
 * tokens and sit at the same position: what Engine.generate builds, one prompt prefilled at batch 1 and its cache copied to every
 * row (nanochat/engine.py:198-214, KVCache.prefill :123-137).  The caches keep the reference's layout and contents, every row
 * holding its copy; the call reads positions [0, shared_len) from row 0 only, once for all rows, on the bf16 matrix cores, and
 * streams per row only the row's own tail [shared_len, p], then merges the two parts of the softmax: the result is that of
 * nc_decode_attention to rounding (sums in another order; the shared part's weights pass through bf16 like in the
 * many-queries kernel), the cache bytes read drop from B x n_keys to shared + B x own.  CONTRACT: rows [0, shared_len) of
 * every batch row hold identical bytes, cache_seqlens[b] is the same for all b and >= shared_len.  workspace:
 * nc_decode_attention_shared_workspace_bytes() bytes, 16-byte aligned.  Any batch size (each row's own tail is read by one workgroup
 * per kv head or head pair).  No counterpart in the reference's attention seam. */
size_t nc_decode_attention_shared_workspace_bytes(int B, int H, int Hkv, int shared_len);
int nc_decode_attention_shared(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache, const int32_t* cache_seqlens,
                               int shared_len, int window_left, uint16_t* out, int B, int H, int Hkv, int Tmax,
                               int seqlens_include_new, void* workspace, size_t workspace_bytes, uint32_t* amax_ws,
                               nc_stream_t stream);

/* nc_decode_attention for callers that cannot allocate device memory and have no workspace to hand over: code under HIP
 * graph capture, tight serving loops, harnesses that forbid allocation.  It has no counterpart in the reference.  Same
 * arguments and results as nc_decode_attention minus the workspace: the split counters and partial results live in a
 * device array built into the library (8.65 MB, held by every GPU the library runs on until the process ends).  Limit:
 * B * T * H <= nc_decode_attention_static_max_row_heads() (1024), larger calls are refused with an error.  The call
 * allocates nothing and clears what it needs itself with a fill kernel.  All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams, two threads) race; serialise them. */
size_t nc_decode_attention_static_max_row_heads(void);
int nc_decode_attention_static(const uint16_t* q, const uint16_t* k_cache, const uint16_t* v_cache,
                               const int32_t* cache_seqlens, int window_left, uint16_t* out, int B, int T, int H, int Hkv,
                               int Tmax, int seqlens_include_new, uint32_t* amax_ws, int splits, nc_stream_t stream);

/* How a decode-attention launch of this shape is laid out (no counterpart in the reference; for tests and tuning):
 * *splits_out = workgroups that share the keys of one (row, kv head); *heads_per_workgroup_out = 1, or 2 when a workgroup
 * streams two neighbouring kv heads.  splits: the caller's request (0 = choose), as passed to the attention calls. */
int nc_decode_attention_plan(int B, int T, int Hkv, int window_left, int Tmax, int splits, int* splits_out /*host*/,
                             int* heads_per_workgroup_out /*host*/);

/* KVCache.prefill: nanochat/engine.py:123-137.  Copies the first n_tokens positions of every (layer, row) of one
 * cache tensor (keys or values), laid out [layers, src_rows, src_tmax, token_bytes], into every row of
 * [layers, dst_rows, dst_tmax, token_bytes]; src_rows is 1 (broadcast over the destination rows, what the Engine
 * does after its batch-1 prefill) or dst_rows.  token_bytes = n_kv_head * head_dim * 2, a multiple of 16. */
int nc_kv_cache_prefill(const void* src, void* dst, int layers, int src_rows, int dst_rows, int src_tmax, int dst_tmax,
                        int n_tokens, int token_bytes, nc_stream_t stream);

/* (5) softcap * tanh(bf16 logits / softcap) -> fp32: nanochat/gpt.py:511-515. */
int nc_softcap(const uint16_t* raw, float* out, int64_t n, float softcap, nc_stream_t stream);

/* (5) Next-token selection: nanochat/engine.py:140-156.  logits fp32 [B,ld]; temperature 0 =>
 * argmax (first index on ties).  Otherwise noise holds Exp(1) draws, [B,k] with top-k (k =
 * min(top_k,V) <= 4096; rank j of the descending top-k list uses noise[b,j]) or [B,V] without
 * (top_k <= 0), and the draw is argmax_j softmax_j / noise_j, which is what torch.multinomial
 * computes.  out_ids int64 [B]. */
int nc_sample(const float* logits, int B, int V, int ld, float temperature, int top_k, const float* noise,
              int64_t* out_ids, nc_stream_t stream);

/* ---- the whole GPT.forward(idx, kv_cache=...) : nanochat/gpt.py:459-524 --------------------- */
typedef struct nc_layer_desc {
    const uint8_t* w_qkv;        /* e4m3 [(H+2Hkv)*128, E]: c_q | c_k | c_v rows (gpt.py:77-79) */
    const float* inv_qkv;        /* fp32 [3]: one inverse scale per stacked weight */
    const uint8_t* w_attn_proj;  /* e4m3 [E, H*128]        (gpt.py:80)  */
    const float* inv_attn_proj;  /* fp32 [1] */
    const uint8_t* w_fc;         /* e4m3 [4E, E]           (gpt.py:134) */
    const float* inv_fc;
    const uint8_t* w_mlp_proj;   /* e4m3 [E, 4E]           (gpt.py:135) */
    const float* inv_mlp_proj;
    const uint16_t* ve_table;    /* bf16 [padded_vocab, Hkv*128] or NULL (gpt.py:192) */
    const float* ve_gate_w;      /* fp32 [Hkv,12] or NULL  (gpt.py:82)  */
    int window_left;             /* gpt.py:287-314 */
    int reserved;
} nc_layer_desc;

typedef struct nc_model_desc {
    int n_layer, n_head, n_kv_head, n_embd, vocab_size, padded_vocab, rope_len, reserved;
    float softcap;
    float reserved_f;
    const uint16_t* wte;         /* bf16 [padded_vocab, E] */
    const uint8_t* w_lm_head;    /* e4m3 [padded_vocab, E] */
    const float* inv_lm_head;    /* fp32 [1] */
    const float* resid_lambdas;  /* fp32 [L] */
    const float* x0_lambdas;     /* fp32 [L] */
    const float* smear_w;        /* fp32 [24] */
    const float* smear_lambda;   /* fp32 [1] */
    const float* backout_lambda; /* fp32 [1] */
    const uint16_t* cos;         /* bf16 [rope_len, 64] */
    const uint16_t* sin;
    const nc_layer_desc* layers; /* HOST array of n_layer entries */
} nc_model_desc;

typedef struct nc_cache_desc {
    uint16_t* k_cache;           /* bf16 [L, B, Tmax, Hkv, 128]  (engine.py:98-99) */
    uint16_t* v_cache;
    const int32_t* cache_seqlens;/* int32 [B], tokens cached before this call; the caller advances it (but see `advance`) */
    const uint16_t* prev_in;     /* bf16 [B,E] or NULL: KVCache.prev_embedding */
    uint16_t* prev_out;          /* bf16 [B,E]: the value to keep for the next call */
    int batch, max_seq_len;
    /* Rows that share their first tokens (optional; 0 = every row reads its own cache everywhere).  shared_prefix > 0 promises that
     * positions [0, shared_prefix) of every batch row hold identical bytes in every layer (KVCache.prefill from a batch-1 cache,
     * nanochat/engine.py:123-137) and that all rows sit at the same position uniform_pos (= cache_seqlens[b] for all b, a host copy)
     * >= shared_prefix.  A one-token-per-row forward then reads the shared keys of full-context layers once for all rows
     * (nc_decode_attention_shared); results equal to rounding, the caches themselves are untouched by the promise. */
    int shared_prefix, uniform_pos;
    /* advance != 0 (one-token forwards only, T = 1): nc_gpt_forward adds it to every row's cache_seqlens itself, inside its last row
     * kernel, once every layer has read the positions; the caller then must not advance them again (saves the caller's own launch,
     * ~5 us of a decode step).  0: the caller advances, as nanochat/gpt.py:122-123 does. */
    int advance;
} nc_cache_desc;

size_t nc_gpt_workspace_bytes(const nc_model_desc* model /*host*/, int B, int T);

/* idx int64 [B,T]; logits_out fp32 [B*T, vocab_size] (all positions) or, with last_only = 1,
 * [B, vocab_size] (the last position of every row, which is all Engine.generate reads).
 * workspace: nc_gpt_workspace_bytes() bytes, 256-byte aligned.  Appends K/V of the T tokens at
 * cache_seqlens[b].. in every layer; the caller then advances cache_seqlens by T (gpt.py:122-123). */
int nc_gpt_forward(const nc_model_desc* model /*host*/, const nc_cache_desc* cache /*host*/, const int64_t* idx,
                   int B, int T, float* logits_out, int last_only, void* workspace, size_t workspace_bytes,
                   nc_stream_t stream);

/* The same forward with its intermediate activations copied out, for layer-by-layer comparison with another implementation
 * (no counterpart in the reference; tests only).  tap_x (or NULL): bf16 [n_layer+1, B*T, E]; slot i is the residual stream as
 * layer i reads it, i.e. after `x = resid_lambdas[i]*x + x0_lambdas[i]*x0` (nanochat/gpt.py:500), slot n_layer the final
 * normalised rows that lm_head reads (gpt.py:508).  tap_y (or NULL): bf16 [n_layer, B*T, H*128], the attention outputs
 * before c_proj (gpt.py:113-124). */
int nc_gpt_forward_tapped(const nc_model_desc* model /*host*/, const nc_cache_desc* cache /*host*/, const int64_t* idx,
                          int B, int T, float* logits_out, int last_only, void* workspace, size_t workspace_bytes,
                          uint16_t* tap_x, uint16_t* tap_y, nc_stream_t stream);

/* ---- measurement aid (no counterpart in the reference) --------------------------------------
 * While enabled, every launch made by this library is bracketed by a HIP event pair on its stream.
 * Classes: 0 attention (partial + combine), 1 FP8 GEMM, 2 quantize/convert, 3 row kernels, 4 sampler, 5 nc_probe_hbm_read.
 * `units` are the algorithmic bytes (classes 0,2,3,4) or flops (class 1) of the launches.  Not thread
 * safe; at most 16384 launches are recorded per enable. */
int nc_profile_enable(int on);
int nc_profile_read(int cls, double* total_ms /*host*/, double* total_units /*host*/, int64_t* count /*host*/);
/* The FP8 GEMM launches (class 1) of one weight shape [N,K] only: the decode step's four linears and lm_head apart. */
int nc_profile_read_gemm(int N, int K, double* total_ms /*host*/, double* total_units /*host*/, int64_t* count /*host*/);

/* What the fp8 matrix cores of this GPU sustain on given operand bytes, with nothing else running (no counterpart in the
 * reference; measurement aid): one 8-wave workgroup per CU issues `iters` rounds of 32 independent
 * v_mfma_f32_16x16x128_f8f6f4 per wave on operands taken once from `operands` (device, e4m3 bytes, 32-byte aligned; NULL =
 * all-zero operands) -- no memory or LDS traffic inside the loop.  The published peak is what all-zero operands reach; the
 * part's power management settles at a lower clock on data whose bits toggle, so an FP8 GEMM on such data is bounded by this
 * figure, not by the published one.  *flops_out (host): flops the launch performs; time it with events.  clocks_out (device,
 * 8 x uint64 or NULL): for workgroups 0..3, shader-clock ticks and 100 MHz ticks spent in the loop (their ratio x 0.1 = GHz). */
int nc_probe_fp8_mfma_ceiling(const uint8_t* operands, int64_t operand_bytes, int iters, uint64_t* clocks_out,
                              double* flops_out /*host*/, nc_stream_t stream);

/* What a kernel that does nothing but read reaches on this GPU's memory (no counterpart in the reference; measurement aid): one
 * launch streams `bytes` of `src` (device, 16-byte aligned) once with 16-byte non-temporal loads and stores nothing.  Time it with
 * events, or enable the profiler above and read class 5 (the kernel's own begin and end); over a buffer larger than the last-level cache its duration is the floor for any kernel that reads as many bytes once.
 * *bytes_read_out (host): the bytes the launch reads (bytes rounded down to a multiple of 16 x the workgroup count). */
int nc_probe_hbm_read(const void* src, int64_t bytes, int64_t* bytes_read_out /*host*/, nc_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif
