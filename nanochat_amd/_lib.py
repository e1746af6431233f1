"""ctypes binding of libnanochat_amd.so (the C ABI of include/nanochat_amd.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnanochat_amd.so")

EXPORTS = [
    "nc_abi_version", "nc_last_error", "nc_fp8_quantize_tensorwise", "nc_e4m3_encode_with_scale", "nc_fp8_gemm_tn",
    "nc_fp8_quantize_tensorwise_as", "nc_fp8_encode_with_scale", "nc_fp8_transpose", "nc_fp8_gemm_tn_grad", "nc_fp8_gemm_tn_relu2",
    "nc_fp8_small_m_workspace_bytes", "nc_fp8_linear_small_m",
    "nc_rmsnorm", "nc_embed_norm_smear", "nc_mix_norm", "nc_relu2", "nc_qkv_rope_append",
    "nc_attention_workspace_bytes", "nc_decode_attention", "nc_kv_cache_prefill", "nc_softcap", "nc_sample",
    "nc_gpt_workspace_bytes", "nc_gpt_forward", "nc_profile_enable", "nc_profile_read", "nc_profile_read_gemm",
    "nc_decode_attention_append", "nc_qkv_rope_append_attention", "nc_decode_attention_plan", "nc_gpt_forward_tapped",
    "nc_decode_attention_static", "nc_decode_attention_static_max_row_heads",
    "nc_fp8_quantize_state_bytes", "nc_fp8_quantize_tensorwise_fused", "nc_fp8_quantize_tensorwise_fused_bounded", "nc_probe_fp8_mfma_ceiling", "nc_probe_hbm_read", "nc_fp8_quantize_tensorwise_transposed",
    "nc_decode_attention_shared", "nc_decode_attention_shared_workspace_bytes",
]


class LayerDesc(C.Structure):
    _fields_ = [("w_qkv", C.c_void_p), ("inv_qkv", C.c_void_p), ("w_attn_proj", C.c_void_p), ("inv_attn_proj", C.c_void_p),
                ("w_fc", C.c_void_p), ("inv_fc", C.c_void_p), ("w_mlp_proj", C.c_void_p), ("inv_mlp_proj", C.c_void_p),
                ("ve_table", C.c_void_p), ("ve_gate_w", C.c_void_p), ("window_left", C.c_int), ("reserved", C.c_int)]


class ModelDesc(C.Structure):
    _fields_ = [("n_layer", C.c_int), ("n_head", C.c_int), ("n_kv_head", C.c_int), ("n_embd", C.c_int),
                ("vocab_size", C.c_int), ("padded_vocab", C.c_int), ("rope_len", C.c_int), ("reserved", C.c_int),
                ("softcap", C.c_float), ("reserved_f", C.c_float),
                ("wte", C.c_void_p), ("w_lm_head", C.c_void_p), ("inv_lm_head", C.c_void_p),
                ("resid_lambdas", C.c_void_p), ("x0_lambdas", C.c_void_p), ("smear_w", C.c_void_p),
                ("smear_lambda", C.c_void_p), ("backout_lambda", C.c_void_p), ("cos", C.c_void_p), ("sin", C.c_void_p),
                ("layers", C.POINTER(LayerDesc))]


class CacheDesc(C.Structure):
    _fields_ = [("k_cache", C.c_void_p), ("v_cache", C.c_void_p), ("cache_seqlens", C.c_void_p),
                ("prev_in", C.c_void_p), ("prev_out", C.c_void_p), ("batch", C.c_int), ("max_seq_len", C.c_int),
                ("shared_prefix", C.c_int), ("uniform_pos", C.c_int), ("advance", C.c_int)]


_lib = None


def _bind(lib):
    p, i, i64, f, sz = C.c_void_p, C.c_int, C.c_int64, C.c_float, C.c_size_t
    sig = {
        "nc_abi_version": (i, []),
        "nc_last_error": (C.c_char_p, []),
        "nc_fp8_quantize_tensorwise": (i, [p, i, i64, p, p, p, p, i, p]),
        "nc_e4m3_encode_with_scale": (i, [p, i64, f, p, i, p]),
        "nc_fp8_quantize_tensorwise_as": (i, [p, i, i64, i, p, p, p, p, i, p]),
        "nc_fp8_quantize_state_bytes": (sz, []),
        "nc_fp8_quantize_tensorwise_fused": (i, [p, i, i64, i, p, p, p, p, i, p]),
        "nc_fp8_quantize_tensorwise_fused_bounded": (i, [p, i, i64, i, p, p, p, p, i, C.c_uint32, p]),
        "nc_fp8_encode_with_scale": (i, [p, i64, f, i, p, i, p]),
        "nc_fp8_transpose": (i, [p, i, i, p, p]),
        "nc_fp8_quantize_tensorwise_transposed": (i, [p, i, i, i, p, p, p, p, p, p]),
        "nc_fp8_gemm_tn_grad": (i, [p, p, p, p, p, i, i, i, i, i, p]),
        "nc_fp8_gemm_tn_relu2": (i, [p, p, p, p, p, p, i, i, i, i, i, p]),
        "nc_fp8_gemm_tn": (i, [p, p, p, p, p, i, p, i, f, i, i, i, i, i, p, sz, p]),
        "nc_fp8_small_m_workspace_bytes": (sz, [i, i, i]),
        "nc_fp8_linear_small_m": (i, [p, p, p, p, p, i, p, i, f, p, i, i, i, i, p, sz, i, p]),
        "nc_rmsnorm": (i, [p, p, i, i, p, p]),
        "nc_embed_norm_smear": (i, [p, p, p, p, p, p, p, i, i, i, i, p]),
        "nc_mix_norm": (i, [p, p, p, p, p, p, p, p, p, i, i, p, p]),
        "nc_relu2": (i, [p, p, i64, p, p]),
        "nc_qkv_rope_append": (i, [p, i, p, i, p, p, p, p, p, i, p, p, p, p, i, i, i, i, i, i, p]),
        "nc_attention_workspace_bytes": (sz, [i, i, i, i]),
        "nc_decode_attention": (i, [p, p, p, p, i, p, i, i, i, i, i, i, p, sz, p, i, p]),
        "nc_decode_attention_append": (i, [p, p, p, p, p, p, i, p, i, i, i, i, i, p, sz, p, i, p]),
        "nc_qkv_rope_append_attention": (i, [p, i, p, i, p, p, p, p, p, i, p, p, p, i, p, i, i, i, i, i, p, sz, p, i, p]),
        "nc_decode_attention_static": (i, [p, p, p, p, i, p, i, i, i, i, i, i, p, i, p]),
        "nc_decode_attention_static_max_row_heads": (sz, []),
        "nc_decode_attention_shared_workspace_bytes": (sz, [i, i, i, i]),
        "nc_decode_attention_shared": (i, [p, p, p, p, i, i, p, i, i, i, i, i, p, sz, p, p]),
        "nc_decode_attention_plan": (i, [i, i, i, i, i, i, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
        "nc_kv_cache_prefill": (i, [p, p, i, i, i, i, i, i, i, p]),
        "nc_softcap": (i, [p, p, i64, f, p]),
        "nc_sample": (i, [p, i, i, i, f, i, p, p, p]),
        "nc_gpt_workspace_bytes": (sz, [C.POINTER(ModelDesc), i, i]),
        "nc_gpt_forward": (i, [C.POINTER(ModelDesc), C.POINTER(CacheDesc), p, i, i, p, i, p, sz, p]),
        "nc_gpt_forward_tapped": (i, [C.POINTER(ModelDesc), C.POINTER(CacheDesc), p, i, i, p, i, p, sz, p, p, p]),
        "nc_profile_enable": (i, [i]),
        "nc_profile_read": (i, [i, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
        "nc_profile_read_gemm": (i, [i, i, C.POINTER(C.c_double), C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
        "nc_probe_fp8_mfma_ceiling": (i, [p, i64, i, p, C.POINTER(C.c_double), p]),
        "nc_probe_hbm_read": (i, [p, i64, C.POINTER(C.c_int64), p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)     # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    return lib


def lib():
    """The loaded library.  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -m nanochat_amd.build` "
                               "(there is no non-HIP fallback)")
        # a rebuild that failed leaves the previous library in place: refuse one whose build stamp names other sources
        from . import build as _build
        if os.path.exists(_build.STAMP_PATH) and open(_build.STAMP_PATH).read().strip() != _build.sources_digest():
            raise RuntimeError(f"{LIB_PATH} was built from other sources than this tree holds: rebuild it with "
                               "`python -m nanochat_amd.build`")
        _lib = _bind(C.CDLL(LIB_PATH))
    return _lib


class NcError(RuntimeError):
    pass


def check(rc):
    """Turn a negative return code into an exception: -1 (bad argument) -> ValueError, else NcError."""
    if rc == 0:
        return
    msg = lib().nc_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(msg)
    raise NcError(f"[{rc}] {msg}")
