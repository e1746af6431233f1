// Internal launch functions shared between the C ABI (nc_api.hip) and the fused forward
// (nc_forward.hip).  Every function enqueues work on the given stream, never synchronises,
// never allocates, and returns 0 or a negative code after nc_set_error().
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;

// ---- quantize (nc_quantize.hip)
void nc_clear_u32(uint32_t* p, int n, hipStream_t s);
int nc_launch_quantize(const void* x, int x_dtype, int64_t n, int fmt, uint8_t* out, float* scale_out, float* inv_out,
                       uint32_t* amax_ws, int encoder, hipStream_t s);
#define NC_QUANTIZE_STATE_BYTES 1536
#define NC_QUANTIZE_DEFAULT_SPINS (1u << 22)      // ~4 M polls of a few hundred ns each before a workgroup stops waiting
int nc_launch_quantize_fused(const void* x, int x_dtype, int64_t n, int fmt, uint8_t* out, float* scale_out, float* inv_out,
                             uint32_t* state, int encoder, hipStream_t s, uint32_t spin_limit = NC_QUANTIZE_DEFAULT_SPINS);
int nc_launch_transpose_u8(const uint8_t* src, int R, int C, uint8_t* dst, hipStream_t s);
int nc_launch_quantize_transposed(const bf16_t* x, int R, int C, int fmt, uint8_t* out, uint8_t* out_t, float* scale_out, float* inv_out,
                                  uint32_t* amax_ws, hipStream_t s);
int nc_launch_convert_only(const void* x, int64_t n, uint8_t* out, float* inv_out, const uint32_t* amax_ws, hipStream_t s);
int nc_launch_encode_with_scale(const bf16_t* x, int64_t n, float scale, int fmt, uint8_t* out, int encoder, hipStream_t s);

// ---- GEMM (nc_gemm.hip)
struct NcGemmSegs {      // column segments of B, each with its own weight inv-scale
    int nseg;
    int end[4];          // exclusive column end of each segment
};
// out_kind: 0 = bf16 [M,ldc];  1 = fp32 [M,ldc] of softcap*tanh(bf16(v)/softcap);  2 = bf16 relu(bf16(v))^2 + amax (M > 128)
int nc_launch_gemm(const uint8_t* a, const uint8_t* b, const float* inv_a, const float* inv_b, NcGemmSegs segs,
                   void* out, int out_kind, float softcap, int M, int N, int K, int ldc, int force_kernel, void* workspace,
                   size_t workspace_bytes, hipStream_t s, int a_fmt = 0,    // a_fmt: 0 e4m3fn, 1 e5m2 (kernels 5, 8, 9)
                   uint32_t* out_amax = nullptr);                            // out_kind 2: bf16 relu(v)^2, amax of it published here

// small-M path (nc_gemm_decode.hip): A is e4m3 (+inv_a) or bf16 (+amax, quantized inside the kernel)
// out_kind: 0 bf16, 1 softcapped fp32, 2 bf16 relu^2 with amax of the result into out_amax.
// With K split over workgroups the raw fp32 sums land in `partials` [ksplits][M][N] and a consumer finishes them.
struct NcRowRecipe;
int nc_gemm_decode_splits(int N, int K);
size_t nc_gemm_decode_partial_bytes(int M, int N, int K);        // any split count up to 16
size_t nc_gemm_decode_partial_bytes_auto(int M, int N, int K);   // the split count nc_gemm_decode_splits() picks
int nc_launch_gemm_decode(const void* a, int a_is_bf16, const uint32_t* a_amax, const float* inv_a, const uint8_t* b,
                          const float* inv_b, NcGemmSegs segs, void* out, int out_kind, float softcap, uint32_t* out_amax, int M,
                          int N, int K, int ldc, float* partials, size_t partial_bytes, int ksplits, int* ksplits_out, hipStream_t s,
                          const NcRowRecipe* recipe = nullptr);     // rows made inside the kernel instead of read from `a`
int nc_launch_finish_partials(const float* parts, int nsplit, const uint32_t* a_amax, const float* inv_a, const float* inv_b,
                              NcGemmSegs segs, void* out, int out_kind, float softcap, uint32_t* out_amax, int M, int N, int ldc,
                              hipStream_t s);

// An FP8 linear's output that still sits in split partials: value(row, col) =
// bf16((sum_s parts[s*split_stride + row*ld + col]) * inv_a * inv_b[segment(col)]), inv_a = 1/scale(amax).
struct NcPartialSrc {
    const float* parts;       // nullptr: not used
    int nsplit;
    int ld;
    size_t split_stride;
    const uint32_t* a_amax;
    const float* inv_b;       // one per segment
    int seg_end0, seg_end1;   // column ends of segments 0 and 1 (INT_MAX when there is a single segment)
};

// How the rows of a small-M linear's input come to be, when the kernel that used to make them is folded into the linear.  For one or
// two rows every workgroup of the GEMM repeats the row arithmetic for itself (a few KB from L2, a few hundred instructions), which
// costs less than the launch it saves; one workgroup also stores what other kernels read (the residual stream, the normalised rows,
// the amax).  The arithmetic and its order are those of mix_norm / finish_partials, so the results are the same bits.
#define NC_RECIPE_MAX_ROWS 2
#define NC_RECIPE_MAX_K 8192
struct NcRowRecipe {
    int kind;                   // 0 none; 1 residual add + lambda mix + norm (mix_norm); 2 relu(.)^2 of a split linear (finish_partials)
    const bf16_t* x_in;         // kind 1: the residual stream [M,K] as it is ...
    bf16_t* x_out;              //         ... and where its new value goes (another buffer: the other workgroups still read x_in)
    const bf16_t* add;          //         a bf16 addend, or
    NcPartialSrc padd;          //         split partial sums to add (kind 2: the linear whose relu^2 the rows are)
    const bf16_t* x0;           //         with resid_lambda / x0_lambda: x = rl * x + xl * x0
    const float* resid_lambda;
    const float* x0_lambda;
    bf16_t* save;               //         copy of x before the lambda mix (the backout rows), or null
    bf16_t* xn_out;             //         the normalised rows, for whoever reads them besides this GEMM
    uint32_t* amax_out;         // the site that receives the amax of the rows
};

// ---- elementwise / norm / rope (nc_elementwise.hip)
int nc_launch_rmsnorm(const bf16_t* x, bf16_t* out, int rows, int cols, uint32_t* amax_ws, hipStream_t s);
int nc_launch_embed_norm_smear(const int64_t* idx, const bf16_t* wte, const float* smear_w, const float* smear_lambda,
                               const bf16_t* prev_in, bf16_t* prev_out, bf16_t* x_out, bf16_t* x0_out, int B, int T, int E,
                               int vocab_rows, uint32_t* clear_words, int n_clear, hipStream_t s);
int nc_launch_mix_norm(bf16_t* x, const bf16_t* add, const bf16_t* x0, const float* resid_lambda, const float* x0_lambda,
                       const float* backout_lambda, const bf16_t* backout_src, bf16_t* backout_save, bf16_t* xn_out,
                       int rows, int cols, uint32_t* amax_ws, hipStream_t s, int32_t* bump = nullptr, int bump_by = 0);
// (bump: int32 [rows] or null; row r's workgroup adds bump_by to bump[r] when it is done -- the cache positions of a decode step)
// same, with the added tensor given as split partials of the linear that produced it (decode path)
int nc_launch_mix_norm_p(bf16_t* x, NcPartialSrc add, const bf16_t* x0, const float* resid_lambda, const float* x0_lambda,
                         const float* backout_lambda, const bf16_t* backout_src, bf16_t* backout_save, bf16_t* xn_out,
                         int rows, int cols, uint32_t* amax_ws, hipStream_t s, int32_t* bump = nullptr, int bump_by = 0);
int nc_launch_relu2(const bf16_t* h, bf16_t* out, int64_t n, uint32_t* amax_ws, hipStream_t s);
int nc_launch_qkv_rope_append_p(NcPartialSrc qkv_parts, const bf16_t* xn, int ld_xn, const int64_t* idx,
                                const bf16_t* ve_table, const float* ve_gate_w, const bf16_t* cos, const bf16_t* sin,
                                int rope_len, const int32_t* cache_seqlens, bf16_t* k_cache, bf16_t* v_cache, bf16_t* q_out,
                                int B, int T, int H, int Hkv, int Tmax, int vocab_rows, hipStream_t s);
int nc_launch_qkv_rope_append(const bf16_t* qkv, int ld_qkv, const bf16_t* xn, int ld_xn, const int64_t* idx,
                              const bf16_t* ve_table, const float* ve_gate_w, const bf16_t* cos, const bf16_t* sin,
                              int rope_len, const int32_t* cache_seqlens, bf16_t* k_cache, bf16_t* v_cache, bf16_t* q_out,
                              int B, int T, int H, int Hkv, int Tmax, int vocab_rows, hipStream_t s);

int nc_launch_kv_prefill_copy(const void* src, void* dst, int layers, int src_rows, int dst_rows, int src_tmax, int dst_tmax,
                              int n_tokens, int token_bytes, hipStream_t s);

// ---- attention (nc_attention.hip)
size_t nc_attn_counter_bytes(int B, int T, int H);
size_t nc_attn_partial_bytes(int B, int T, int H);
int nc_launch_attention(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens,
                        int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                        uint32_t* counters, void* partials, size_t partial_bytes, uint32_t* amax_ws, int force_splits,
                        int counters_are_zero, hipStream_t s);

// many query positions per row (nc_attention_prefill.hip): flash-attention forward on the bf16 matrix cores
// compute units of the current device (looked up once per process and device)
int nc_cu_count();
int nc_launch_attention_prefill(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens,
                                int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new,
                                uint32_t* amax_ws, hipStream_t s);
int nc_attn_splits(int B, int T, int Hkv, int window_left, int Tmax);
// rows that share their first cached tokens (nc_attention_prefill.hip, nc_attention.hip)
void nc_attn_shared_plan(int rows, int H, int Hkv, int shared_len, int* chunk_keys_out, int* nchunks_out);
size_t nc_attn_shared_partial_bytes(int rows, int H, int Hkv, int shared_len);
int nc_launch_attention_shared_prefix(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int shared_len,
                                      int window_left, int seqlens_include_new, float* partials, size_t partial_bytes, int rows, int H, int Hkv,
                                      int Tmax, int* nchunks_out, hipStream_t s);
int nc_launch_attention_shared(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int shared_len,
                               int window_left, bf16_t* out, int B, int H, int Hkv, int Tmax, int seqlens_include_new, void* shared_parts,
                               size_t shared_part_bytes, uint32_t* amax_ws, hipStream_t s);
void nc_attention_plan(int B, int T, int Hkv, int window_left, int Tmax, int force_splits, int* splits_out, int* heads_per_wg_out);
int nc_launch_attention_append(const bf16_t* q, const bf16_t* k_new, const bf16_t* v_new, bf16_t* k_cache, bf16_t* v_cache,
                               const int32_t* cache_seqlens, int window_left, bf16_t* out, int B, int T, int H, int Hkv, int Tmax,
                               uint32_t* counters, void* partials, size_t partial_bytes, uint32_t* amax_ws, int force_splits,
                               hipStream_t s);
size_t nc_attention_static_max_row_heads(void);
int nc_launch_attention_static(const bf16_t* q, const bf16_t* k_cache, const bf16_t* v_cache, const int32_t* cache_seqlens, int window_left,
                               bf16_t* out, int B, int T, int H, int Hkv, int Tmax, int seqlens_include_new, uint32_t* amax_ws,
                               int force_splits, hipStream_t s);
struct NcRopeSrc;
int nc_launch_attention_fused(NcRopeSrc rope, bf16_t* k_cache, bf16_t* v_cache, const int32_t* cache_seqlens, int window_left,
                              bf16_t* out, int B, int H, int Hkv, int Tmax, uint32_t* counters, void* partials, size_t partial_bytes,
                              uint32_t* amax_ws, int force_splits, int counters_are_zero, hipStream_t s);

// ---- sampling (nc_sample.hip)
int nc_launch_softcap(const bf16_t* raw, float* out, int64_t n, float softcap, hipStream_t s);
int nc_launch_sample(const float* logits, int B, int V, int ld, float temperature, int top_k, const float* noise,
                     int64_t* out_ids, hipStream_t s);

// ---- optional event timing (nc_profile.hip)
int nc_prof_begin(int cls, double units, hipStream_t s, int64_t tag = 0);
void nc_prof_end(int slot, hipStream_t s);
bool nc_prof_take(int cls, double units, int64_t tag, hipEvent_t* start, hipEvent_t* stop);
struct NcProfScope {
    int slot;
    hipStream_t s;
    NcProfScope(int cls, double units, hipStream_t st, int64_t tag = 0) : slot(nc_prof_begin(cls, units, st, tag)), s(st) {}
    ~NcProfScope() { nc_prof_end(slot, s); }
};
