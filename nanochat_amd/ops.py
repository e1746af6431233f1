"""Tensor-level wrappers over the C ABI: validate, hand raw device pointers and the current HIP
stream to libnanochat_amd.so, return torch tensors.  torch is used for memory and streams only.

Every function requires CUDA (ROCm) tensors and raises otherwise: there is no CPU path here.
"""
import ctypes as C

import torch

from . import _lib

_SCRATCH = {}


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _need_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("nanochat_amd ops run on the GPU only (got a CPU tensor); there is no CPU fallback")


def _quantize_state(device):
    """The quantizer's state block (zero before first use, left zero by every call), one per device and stream."""
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    t = _SCRATCH.get(key)
    if t is None:
        nbytes = _lib.lib().nc_fp8_quantize_state_bytes()
        raw = torch.zeros(nbytes + 128, dtype=torch.uint8, device=device)
        off = (-raw.data_ptr()) % 128
        t = raw[off:off + nbytes]
        _SCRATCH[key] = t
    return t


# ----------------------------------------------------------------------------- (1) quantize
_FP8_FORMATS = {torch.float8_e4m3fn: 0, torch.float8_e5m2: 1}


QUANTIZE_SLOW_WORD = 257      # uint32 index in the quantizer's state block: workgroups that ever took the slow way (sticky)


def quantize_slow_count(device=None):
    """How many workgroups of the one-launch quantizer ever gave up waiting for their peers on this device and stream, and worked
    the amax out alone (correct results, slowly): non-zero means more such grids overlapped on the GPU than it holds at once.
    Reads the device (a synchronisation); for diagnostics and tests."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    return int(_quantize_state(device).view(torch.int32)[QUANTIZE_SLOW_WORD].item())


def fp8_quantize(x, encoder=0, fp8_dtype=torch.float8_e4m3fn, spin_limit=None):
    """Tensorwise fp8 quantization of a bf16/fp32 tensor (nanochat/fp8.py:81-107): e4m3fn, or e5m2 for gradients.

    Returns (payload of fp8_dtype with x's shape, inv_scale fp32 0-dim, scale fp32 0-dim).  spin_limit (tests): the bound of the
    one-launch kernel's wait for its peers, in polls; None = the library's default."""
    _need_cuda(x)
    if x.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"fp8_quantize: dtype {x.dtype} not supported (bf16 or fp32)")
    if fp8_dtype not in _FP8_FORMATS:
        raise ValueError(f"fp8_quantize: format {fp8_dtype} not supported (float8_e4m3fn or float8_e5m2)")
    x = x.contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scales = torch.empty(2, dtype=torch.float32, device=x.device)
    state = _quantize_state(x.device)
    args = (_ptr(x), 0 if x.dtype == torch.bfloat16 else 1, x.numel(), _FP8_FORMATS[fp8_dtype], _ptr(out), C.c_void_p(scales.data_ptr()),
            C.c_void_p(scales.data_ptr() + 4), _ptr(state), encoder)
    if spin_limit is None:
        rc = _lib.lib().nc_fp8_quantize_tensorwise_fused(*args, _stream())
    else:
        rc = _lib.lib().nc_fp8_quantize_tensorwise_fused_bounded(*args, int(spin_limit), _stream())
    _lib.check(rc)
    return out.view(fp8_dtype), scales[1], scales[0]


def fp8_quantize_transposed(x, fp8_dtype=torch.float8_e4m3fn):
    """Tensorwise fp8 quantization of a bf16 matrix [R,C] that also writes the transposed payload [C,R] from the same read (what the
    backward GEMMs of nanochat/fp8.py:156-192 take: grad_output both ways, the saved input transposed).

    Returns (payload [R,C], payload_t [C,R], inv_scale fp32 0-dim, scale fp32 0-dim); the bits are those of fp8_quantize."""
    _need_cuda(x)
    if x.dtype != torch.bfloat16 or x.dim() != 2:
        raise ValueError("fp8_quantize_transposed: a 2-D bf16 tensor is required")
    if fp8_dtype not in _FP8_FORMATS:
        raise ValueError(f"fp8_quantize_transposed: format {fp8_dtype} not supported (float8_e4m3fn or float8_e5m2)")
    x = x.contiguous()
    R, Cc = x.shape
    out = torch.empty(R, Cc, dtype=torch.uint8, device=x.device)
    out_t = torch.empty(Cc, R, dtype=torch.uint8, device=x.device)
    scales = torch.empty(2, dtype=torch.float32, device=x.device)
    state = _quantize_state(x.device)
    scratch = C.c_void_p(state.data_ptr() + 4 * 320)          # the state block's scratch word
    _lib.check(_lib.lib().nc_fp8_quantize_tensorwise_transposed(_ptr(x), R, Cc, _FP8_FORMATS[fp8_dtype], _ptr(out), _ptr(out_t),
                                                                C.c_void_p(scales.data_ptr()), C.c_void_p(scales.data_ptr() + 4), scratch,
                                                                _stream()))
    return out.view(fp8_dtype), out_t.view(fp8_dtype), scales[1], scales[0]


def fp8_encode_with_scale(x_bf16, scale, fp8_dtype, encoder=0):
    """The saturating cast alone, with a given scale (nanochat/fp8.py:100-103); returns uint8 payload bytes."""
    _need_cuda(x_bf16)
    assert x_bf16.dtype == torch.bfloat16
    x = x_bf16.contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib().nc_fp8_encode_with_scale(_ptr(x), x.numel(), float(scale), _FP8_FORMATS[fp8_dtype], _ptr(out), encoder, _stream()))
    return out


def fp8_transpose(x8):
    """[R,C] fp8 payload -> [C,R] contiguous (the rearrangement of _to_col_major / .t().contiguous(), nanochat/fp8.py:110-118)."""
    _need_cuda(x8)
    if x8.dim() != 2 or x8.element_size() != 1:
        raise ValueError("fp8_transpose: a 2-D one-byte tensor is required")
    x8 = x8.contiguous()
    R, Cc = x8.shape
    out = torch.empty(Cc, R, dtype=x8.dtype, device=x8.device)
    _lib.check(_lib.lib().nc_fp8_transpose(_ptr(x8), R, Cc, _ptr(out), _stream()))
    return out


def fp8_gemm_grad(a_e5m2, w8, inv_a, inv_w, kernel=0, out=None):
    """out[M,N] = bf16((a_e5m2[M,K] @ w8[N,K]^T, fp32 acc) * inv_a * inv_w): the backward GEMMs of nanochat/fp8.py:166-190,
    first operand in e5m2, second in e4m3fn, the summed index contiguous in both."""
    _need_cuda(a_e5m2, w8, inv_a, inv_w)
    if a_e5m2.dim() != 2 or w8.dim() != 2 or a_e5m2.shape[1] != w8.shape[1]:
        raise ValueError(f"fp8_gemm_grad: shapes {tuple(a_e5m2.shape)} x {tuple(w8.shape)}^T do not match")
    if a_e5m2.element_size() != 1 or w8.element_size() != 1:
        raise ValueError("fp8_gemm_grad: operands must be fp8 (one byte per element)")
    a_e5m2, w8 = a_e5m2.contiguous(), w8.contiguous()
    M, K = a_e5m2.shape
    N = w8.shape[0]
    inv_a = inv_a.reshape(-1).float()
    inv_w = inv_w.reshape(-1).float()
    if out is None:
        out = torch.empty(M, N, dtype=torch.bfloat16, device=a_e5m2.device)
    _lib.check(_lib.lib().nc_fp8_gemm_tn_grad(_ptr(a_e5m2), _ptr(w8), _ptr(inv_a), _ptr(inv_w), _ptr(out), M, N, K, out.stride(0), kernel,
                                              _stream()))
    return out


def e4m3_encode_with_scale(x_bf16, scale, encoder=0):
    _need_cuda(x_bf16)
    assert x_bf16.dtype == torch.bfloat16
    x = x_bf16.contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib().nc_e4m3_encode_with_scale(_ptr(x), x.numel(), float(scale), _ptr(out), encoder, _stream()))
    return out


# ----------------------------------------------------------------------------- (2) GEMM
_GEMM_WS = {}


def _small_m_workspace(device, M, N, K):
    """Zero-initialised split-K scratch, kept per device and stream (its counter block stays zero between calls)."""
    need = _lib.lib().nc_fp8_small_m_workspace_bytes(M, N, K)
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    ws = _GEMM_WS.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.zeros(max(need, 1 << 20), dtype=torch.uint8, device=device)
        _GEMM_WS[key] = ws
    return ws


def fp8_gemm(a8, w8, inv_a, inv_w, seg_ends=None, softcap=None, kernel=0, out=None):
    """out[M,N] = bf16((a8[M,K] @ w8[N,K]^T, fp32 acc) * inv_a * inv_w[segment]) (nanochat/fp8.py:143-153).

    inv_w may hold several scales when w8 stacks weights along N; seg_ends lists their column ends.
    With softcap, the result is fp32 softcap*tanh(bf16(v)/softcap) instead."""
    _need_cuda(a8, w8, inv_a, inv_w)
    if a8.dim() != 2 or w8.dim() != 2 or a8.shape[1] != w8.shape[1]:
        raise ValueError(f"fp8_gemm: shapes {tuple(a8.shape)} x {tuple(w8.shape)}^T do not match")
    if a8.element_size() != 1 or w8.element_size() != 1:
        raise ValueError("fp8_gemm: operands must be e4m3 (one byte per element)")
    a8, w8 = a8.contiguous(), w8.contiguous()
    M, K = a8.shape
    N = w8.shape[0]
    inv_a = inv_a.reshape(-1).float()
    inv_w = inv_w.reshape(-1).float().contiguous()
    if seg_ends is None:
        seg_ends = [N]
    if len(seg_ends) != inv_w.numel():
        raise ValueError("fp8_gemm: one weight inverse scale per column segment is required")
    segs = (C.c_int32 * len(seg_ends))(*seg_ends)
    if out is None:
        out = torch.empty(M, N, dtype=torch.float32 if softcap is not None else torch.bfloat16, device=a8.device)
    ws = _small_m_workspace(a8.device, M, N, K) if 1 <= M <= 128 else None
    rc = _lib.lib().nc_fp8_gemm_tn(_ptr(a8), _ptr(w8), _ptr(inv_a), _ptr(inv_w), segs, len(seg_ends), _ptr(out),
                                   1 if softcap is not None else 0, float(softcap or 0.0), M, N, K, out.stride(0), kernel,
                                   _ptr(ws), ws.numel() if ws is not None else 0, _stream())
    _lib.check(rc)
    return out


def fp8_gemm_relu2(a8, w8, inv_a, inv_w, kernel=0):
    """relu(a8 @ w8^T * scales)^2 in bf16 for M > 128 rows, and an int32 tensor with the fp32 bits of its maximum
    (nanochat/gpt.py:138-139 with the amax of the next quantization fused in)."""
    _need_cuda(a8, w8, inv_a, inv_w)
    a8, w8 = a8.contiguous(), w8.contiguous()
    M, K = a8.shape
    N = w8.shape[0]
    out = torch.empty(M, N, dtype=torch.bfloat16, device=a8.device)
    amax = torch.zeros(1, dtype=torch.int32, device=a8.device)
    _lib.check(_lib.lib().nc_fp8_gemm_tn_relu2(_ptr(a8), _ptr(w8), _ptr(inv_a.reshape(-1).float()), _ptr(inv_w.reshape(-1).float()),
                                               _ptr(out), _ptr(amax), M, N, K, out.stride(0), kernel, _stream()))
    return out, amax


def fp8_linear_small_m(a_bf16, amax_bits, w8, inv_w, seg_ends=None, softcap=None, relu2=False, ksplits=0):
    """Float8Linear.forward for M <= 128 rows in one launch: a_bf16 [M,K] is quantized inside the GEMM with the
    tensorwise scale of amax_bits (int32 tensor holding the fp32 bits of max|a|).  Returns the output, and with
    relu2=True also an int32 tensor with the fp32 bits of max(relu(out)^2)."""
    _need_cuda(a_bf16, amax_bits, w8, inv_w)
    assert a_bf16.dtype == torch.bfloat16 and a_bf16.dim() == 2
    a = a_bf16.contiguous()
    w8 = w8.contiguous()
    M, K = a.shape
    N = w8.shape[0]
    inv_w = inv_w.reshape(-1).float().contiguous()
    if seg_ends is None:
        seg_ends = [N]
    segs = (C.c_int32 * len(seg_ends))(*seg_ends)
    kind = 1 if softcap is not None else (2 if relu2 else 0)
    out = torch.empty(M, N, dtype=torch.float32 if kind == 1 else torch.bfloat16, device=a.device)
    out_amax = torch.zeros(1, dtype=torch.int32, device=a.device) if relu2 else None
    ws = _small_m_workspace(a.device, M, N, K)
    rc = _lib.lib().nc_fp8_linear_small_m(_ptr(a), _ptr(amax_bits), _ptr(w8), _ptr(inv_w), segs, len(seg_ends), _ptr(out), kind,
                                          float(softcap or 0.0), _ptr(out_amax), M, N, K, out.stride(0), _ptr(ws), ws.numel(),
                                          ksplits, _stream())
    _lib.check(rc)
    return (out, out_amax) if relu2 else out


def amax_bits(x):
    """fp32 bit pattern of max|x| as a one-element int32 tensor (what the producer kernels leave in an amax slot)."""
    return x.detach().abs().max().float().reshape(1).view(torch.int32)


# ----------------------------------------------------------------------------- (4) norm / rope / append
def rms_norm(x):
    """Parameter-free RMSNorm over the last dim of a bf16 tensor (nanochat/gpt.py:42-43)."""
    _need_cuda(x)
    if x.dtype != torch.bfloat16:
        raise ValueError("rms_norm: bf16 only on the GPU path")
    x = x.contiguous()
    out = torch.empty_like(x)
    cols = x.shape[-1]
    _lib.check(_lib.lib().nc_rmsnorm(_ptr(x), _ptr(out), x.numel() // cols, cols, C.c_void_p(0), _stream()))
    return out


def relu2(h):
    _need_cuda(h)
    h = h.contiguous()
    out = torch.empty_like(h)
    _lib.check(_lib.lib().nc_relu2(_ptr(h), _ptr(out), h.numel(), C.c_void_p(0), _stream()))
    return out


def embed_norm_smear(idx, wte, smear_w, smear_lambda, prev):
    """(x [B,T,E], new prev_embedding [B,1,E]) -- nanochat/gpt.py:471-492."""
    _need_cuda(idx, wte)
    B, T = idx.shape
    E = wte.shape[1]
    x = torch.empty(B, T, E, dtype=torch.bfloat16, device=idx.device)
    prev_out = torch.empty(B, 1, E, dtype=torch.bfloat16, device=idx.device)
    rc = _lib.lib().nc_embed_norm_smear(_ptr(idx.contiguous()), _ptr(wte), _ptr(smear_w.float().contiguous()),
                                        _ptr(smear_lambda.float().contiguous()), _ptr(prev), _ptr(prev_out), _ptr(x), B, T, E,
                                        wte.shape[0], _stream())
    _lib.check(rc)
    return x, prev_out


def mix_norm(x, add=None, x0=None, resid_lambda=None, x0_lambda=None, backout_lambda=None, backout_src=None,
             want_backout=False):
    """In-place residual update of x plus RMSNorm; returns (xn, saved_rows or None).  See nc_mix_norm."""
    _need_cuda(x)
    assert x.is_contiguous() and x.dtype == torch.bfloat16
    cols = x.shape[-1]
    rows = x.numel() // cols
    xn = torch.empty_like(x)
    saved = torch.empty_like(x) if want_backout else None
    rc = _lib.lib().nc_mix_norm(_ptr(x), _ptr(add), _ptr(x0), _ptr(resid_lambda), _ptr(x0_lambda), _ptr(backout_lambda),
                                _ptr(backout_src), _ptr(saved), _ptr(xn), rows, cols, C.c_void_p(0), _stream())
    _lib.check(rc)
    return xn, saved


def qkv_rope_append(qkv, xn, idx, ve_table, ve_gate_w, cos, sin, cache_seqlens, k_cache, v_cache, n_head, n_kv_head):
    """Rotary + QK-norm + gain on q,k; value-embedding gate on v; append k,v at cache_seqlens.. (in place).
    qkv [B,T,(H+2Hkv)*128] bf16.  Returns q [B,T,H,128]."""
    _need_cuda(qkv, k_cache, v_cache, cache_seqlens)
    B, T = qkv.shape[0], qkv.shape[1]
    qkv = qkv.contiguous()
    q = torch.empty(B, T, n_head, 128, dtype=torch.bfloat16, device=qkv.device)
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    Tmax = k_cache.shape[1]
    vocab_rows = ve_table.shape[0] if ve_table is not None else 0
    xn_c = xn.contiguous() if xn is not None else None
    rc = _lib.lib().nc_qkv_rope_append(_ptr(qkv), qkv.shape[-1], _ptr(xn_c), xn_c.shape[-1] if xn_c is not None else 0,
                                       _ptr(idx.contiguous() if idx is not None else None), _ptr(ve_table),
                                       _ptr(ve_gate_w.float().contiguous() if ve_gate_w is not None else None),
                                       _ptr(cos), _ptr(sin), cos.shape[0], _ptr(cache_seqlens), _ptr(k_cache), _ptr(v_cache),
                                       _ptr(q), B, T, n_head, n_kv_head, Tmax, vocab_rows, _stream())
    _lib.check(rc)
    return q


# ----------------------------------------------------------------------------- (3) attention
def decode_attention(q, k_cache, v_cache, cache_seqlens, window_left=-1, seqlens_include_new=False, splits=0):
    """Attention of q [B,T,H,128] over caches [B,Tmax,Hkv,128] whose new tokens are already appended."""
    _need_cuda(q, k_cache, v_cache, cache_seqlens)
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise ValueError("decode_attention: bf16 only")
    if q.shape[-1] != 128 or k_cache.shape[-1] != 128:
        raise ValueError("decode_attention: head_dim must be 128")
    if cache_seqlens.dtype != torch.int32:
        raise ValueError("decode_attention: cache_seqlens must be int32")
    B, T, H, D = q.shape
    Tmax, Hkv = k_cache.shape[1], k_cache.shape[2]
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("decode_attention: caches must be contiguous (B,Tmax,Hkv,128)")
    q = q.contiguous()
    out = torch.empty_like(q)
    lib = _lib.lib()
    ws, ws_bytes = _attention_workspace(B, T, H, Tmax, q.device)
    rc = lib.nc_decode_attention(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(cache_seqlens), int(window_left), _ptr(out), B, T, H,
                                 Hkv, Tmax, 1 if seqlens_include_new else 0, _ptr(ws), ws_bytes, C.c_void_p(0), splits,
                                 _stream())
    _lib.check(rc)
    return out


def decode_attention_shared(q, k_cache, v_cache, cache_seqlens, shared_len, window_left=-1, seqlens_include_new=False):
    """decode_attention for a batch whose rows all begin with the same `shared_len` cached tokens and sit at the same position (one
    prompt replicated by KVCache.prefill): the shared keys are read once for all rows, each row streams only its own tail."""
    _need_cuda(q, k_cache, v_cache, cache_seqlens)
    if q.dtype != torch.bfloat16 or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16:
        raise ValueError("decode_attention_shared: bf16 only")
    if cache_seqlens.dtype != torch.int32:
        raise ValueError("decode_attention_shared: cache_seqlens must be int32")
    B, T, H, D = q.shape
    Tmax, Hkv = k_cache.shape[1], k_cache.shape[2]
    if T != 1 or D != 128 or k_cache.shape[-1] != 128:
        raise ValueError("decode_attention_shared: one new token per row, head_dim 128")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("decode_attention_shared: caches must be contiguous (B,Tmax,Hkv,128)")
    q = q.contiguous()
    out = torch.empty_like(q)
    lib = _lib.lib()
    ws_bytes = lib.nc_decode_attention_shared_workspace_bytes(B, H, Hkv, int(shared_len))
    key = (q.device.index, torch.cuda.current_stream().cuda_stream, "shared")
    ws = _ATTN_WS.get(key)
    if ws is None or ws.numel() < ws_bytes:
        ws = torch.empty(max(ws_bytes, 1 << 20), dtype=torch.uint8, device=q.device)
        _ATTN_WS[key] = ws
    rc = lib.nc_decode_attention_shared(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(cache_seqlens), int(shared_len), int(window_left), _ptr(out),
                                        B, H, Hkv, Tmax, 1 if seqlens_include_new else 0, _ptr(ws), ws.numel(), C.c_void_p(0), _stream())
    _lib.check(rc)
    return out


_ATTN_WS = {}


def _attention_workspace(B, T, H, Tmax, device):
    """Split counters and partial results of the stand-alone attention entries, kept per device and stream and grown on demand
    (calls on one stream run one after the other, and every call clears its own counters)."""
    ws_bytes = _lib.lib().nc_attention_workspace_bytes(B, T, H, Tmax)
    key = (device.index, torch.cuda.current_stream().cuda_stream)
    ws = _ATTN_WS.get(key)
    if ws is None or ws.numel() < ws_bytes:
        ws = torch.empty(max(ws_bytes, 1 << 20), dtype=torch.uint8, device=device)
        _ATTN_WS[key] = ws
    return ws, ws_bytes


def decode_attention_append(q, k_new, v_new, k_cache, v_cache, cache_seqlens, window_left=-1, splits=0):
    """flash_attn_with_kvcache(q, k_cache, v_cache, k=k_new, v=v_new, cache_seqlens=...) (nanochat/flash_attention.py:139-185):
    the new keys and values go into the caches at cache_seqlens[b].. (in place), then q [B,T,H,128] attends."""
    _need_cuda(q, k_new, v_new, k_cache, v_cache, cache_seqlens)
    for t in (q, k_new, v_new, k_cache, v_cache):
        if t.dtype != torch.bfloat16:
            raise ValueError("decode_attention_append: bf16 only")
    if cache_seqlens.dtype != torch.int32:
        raise ValueError("decode_attention_append: cache_seqlens must be int32")
    B, T, H, D = q.shape
    Tmax, Hkv = k_cache.shape[1], k_cache.shape[2]
    if D != 128 or k_cache.shape[-1] != 128 or tuple(k_new.shape) != (B, T, Hkv, 128) or tuple(v_new.shape) != (B, T, Hkv, 128):
        raise ValueError("decode_attention_append: q [B,T,H,128], k/v [B,T,Hkv,128], caches [B,Tmax,Hkv,128] expected")
    if not (k_cache.is_contiguous() and v_cache.is_contiguous()):
        raise ValueError("decode_attention_append: caches must be contiguous (B,Tmax,Hkv,128)")
    q, k_new, v_new = q.contiguous(), k_new.contiguous(), v_new.contiguous()
    out = torch.empty_like(q)
    ws, ws_bytes = _attention_workspace(B, T, H, Tmax, q.device)
    rc = _lib.lib().nc_decode_attention_append(_ptr(q), _ptr(k_new), _ptr(v_new), _ptr(k_cache), _ptr(v_cache), _ptr(cache_seqlens),
                                               int(window_left), _ptr(out), B, T, H, Hkv, Tmax, _ptr(ws), ws_bytes, C.c_void_p(0),
                                               splits, _stream())
    _lib.check(rc)
    return out


def qkv_rope_append_attention(qkv, xn, idx, ve_table, ve_gate_w, cos, sin, cache_seqlens, k_cache, v_cache, n_head, n_kv_head,
                              window_left=-1, splits=0):
    """Decode (one new token per row): qkv_rope_append and decode_attention in one launch (nanochat/gpt.py:89-120).
    qkv [B,1,(H+2Hkv)*128] bf16.  Returns the attention output [B,1,H,128]; the caches get the new key and value."""
    _need_cuda(qkv, k_cache, v_cache, cache_seqlens)
    B = qkv.shape[0]
    if qkv.numel() != B * (n_head + 2 * n_kv_head) * 128:
        raise ValueError("qkv_rope_append_attention: one new token per row expected")
    qkv = qkv.contiguous()
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    Tmax = k_cache.shape[1]
    out = torch.empty(B, 1, n_head, 128, dtype=torch.bfloat16, device=qkv.device)
    vocab_rows = ve_table.shape[0] if ve_table is not None else 0
    xn_c = xn.contiguous() if xn is not None else None
    ws, ws_bytes = _attention_workspace(B, 1, n_head, Tmax, qkv.device)
    rc = _lib.lib().nc_qkv_rope_append_attention(
        _ptr(qkv), qkv.shape[-1], _ptr(xn_c), xn_c.shape[-1] if xn_c is not None else 0, _ptr(idx.contiguous() if idx is not None else None),
        _ptr(ve_table), _ptr(ve_gate_w.float().contiguous() if ve_gate_w is not None else None), _ptr(cos), _ptr(sin), cos.shape[0],
        _ptr(cache_seqlens), _ptr(k_cache), _ptr(v_cache), int(window_left), _ptr(out), B, n_head, n_kv_head, Tmax, vocab_rows,
        _ptr(ws), ws_bytes, C.c_void_p(0), splits, _stream())
    _lib.check(rc)
    return out


def decode_attention_plan(B, T, n_kv_head, window_left, Tmax, splits=0):
    """(key splits, kv heads per workgroup) a decode-attention launch of this shape uses."""
    s, h = C.c_int(0), C.c_int(0)
    _lib.check(_lib.lib().nc_decode_attention_plan(B, T, n_kv_head, int(window_left), Tmax, splits, C.byref(s), C.byref(h)))
    return s.value, h.value


def kv_cache_prefill(dst, src, n_tokens):
    """dst[:, :, :n] = src[:, :, :n] for cache tensors (L, B, T, Hkv, D); a one-row src is broadcast (engine.py:129-130)."""
    _need_cuda(dst, src)
    if not (dst.is_contiguous() and src.is_contiguous() and dst.dtype == src.dtype == torch.bfloat16):
        raise ValueError("kv_cache_prefill: contiguous bf16 cache tensors expected")
    L, Bd, Td, Hkv, D = dst.shape
    Ls, Bs, Ts, Hs, Ds = src.shape
    if (Ls, Hs, Ds) != (L, Hkv, D):
        raise ValueError("kv_cache_prefill: layer / head geometry differs")
    _lib.check(_lib.lib().nc_kv_cache_prefill(_ptr(src), _ptr(dst), L, Bs, Bd, Ts, Td, int(n_tokens), Hkv * D * 2, _stream()))


# ----------------------------------------------------------------------------- (5) softcap / sample
def softcap(raw_bf16, cap=15.0):
    _need_cuda(raw_bf16)
    raw = raw_bf16.contiguous()
    out = torch.empty(raw.shape, dtype=torch.float32, device=raw.device)
    _lib.check(_lib.lib().nc_softcap(_ptr(raw), _ptr(out), raw.numel(), float(cap), _stream()))
    return out


def sample(logits, temperature, top_k, noise=None):
    """Next-token ids [B,1] from fp32 logits [B,V] (nanochat/engine.py:140-156); noise: Exp(1) draws."""
    _need_cuda(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise ValueError("sample: logits must be fp32 [B,V]")
    if logits.stride(1) != 1 or logits.stride(0) < logits.shape[1]:
        logits = logits.contiguous()
    B, V = logits.shape
    out = torch.empty(B, 1, dtype=torch.int64, device=logits.device)
    k = 0 if (top_k is None or top_k <= 0) else min(int(top_k), V)
    if noise is not None:
        noise = noise.contiguous()
        want = k if (0 < k < V) else V
        if tuple(noise.shape) != (B, want):
            raise ValueError(f"sample: noise must have shape {(B, want)}, got {tuple(noise.shape)}")
    rc = _lib.lib().nc_sample(_ptr(logits), B, V, logits.stride(0), float(temperature), k, _ptr(noise), _ptr(out), _stream())
    _lib.check(rc)
    return out
