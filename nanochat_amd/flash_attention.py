"""The attention plug-in seam of nanochat (nanochat/flash_attention.py:191-195), served by the HIP
split-K kernel instead of FA3 / SDPA.

    from nanochat_amd.flash_attention import flash_attn
    y = flash_attn.flash_attn_with_kvcache(q, k_cache, v_cache, k=k, v=v, cache_seqlens=..., causal=True,
                                           window_size=(w, 0))

Layouts are FA3's: q (B,T,H,D), caches (B,Tmax,Hkv,D), D = 128, bf16.  The cache is updated in place
and cache_seqlens is NOT advanced (the caller does that, nanochat/gpt.py:122-123).  Unlike the SDPA
fallback of the reference (flash_attention.py:165) every row uses its own cache_seqlens entry.
"""
from types import SimpleNamespace

import torch

from . import ops


def flash_attn_with_kvcache(q, k_cache, v_cache, k=None, v=None, cache_seqlens=None, causal=False,
                            window_size=(-1, -1)):
    assert cache_seqlens is not None, "cache_seqlens is required"
    assert causal, "only causal attention is implemented (nanochat always passes causal=True)"
    if k is not None and v is not None:
        # in-place insert at [pos_b, pos_b + T) per row (flash_attention.py:167-170), done by the library
        return ops.decode_attention_append(q, k.to(k_cache.dtype), v.to(v_cache.dtype), k_cache, v_cache, cache_seqlens,
                                           window_left=window_size[0])
    return ops.decode_attention(q, k_cache, v_cache, cache_seqlens, window_left=window_size[0])


def flash_attn_func(q, k, v, causal=False, window_size=(-1, -1)):
    """Cache-free causal attention (flash_attention.py:115-136), forward only: the sequence is its own cache."""
    assert causal, "only causal attention is implemented"
    B = q.shape[0]
    zeros = torch.zeros(B, dtype=torch.int32, device=q.device)
    return ops.decode_attention(q, k.contiguous(), v.contiguous(), zeros, window_left=window_size[0])


flash_attn = SimpleNamespace(flash_attn_func=flash_attn_func, flash_attn_with_kvcache=flash_attn_with_kvcache)
