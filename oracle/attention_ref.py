"""Oracle: KV-cache attention with causal mask, left sliding window and GQA.

Test infrastructure only; never imported by the product package.

Semantics follow the SDPA branch of nanochat/flash_attention.py:139-185 with the
masks of :77-110, generalised to per-row ``cache_seqlens`` (which the FA3
signature at :157-161 carries, but the SDPA fallback collapses to row 0 at :165).
Layouts: q [B,Tn,H,D]; k_cache/v_cache [B,Tmax,Hkv,D]; k/v [B,Tn,Hkv,D].
"""
import math
import torch
import torch.nn.functional as F


def key_range(pos, t, window_left):
    """Keys visible to the query at new-token index t of a row whose cache held
    ``pos`` tokens: [lo, hi] inclusive.  Causal: hi = pos+t.  Left window w:
    the last w+1 keys (flash_attention.py:91-97, tests/test_attention_fallback.py:182-213)."""
    hi = pos + t
    lo = 0 if window_left < 0 else max(0, hi - window_left)
    return lo, hi


def attention_with_kvcache(q, k_cache, v_cache, k=None, v=None, cache_seqlens=None,
                           window_size=(-1, 0), math_dtype=torch.float32):
    """In-place cache append followed by masked softmax attention.

    Returns [B,Tn,H,D] in q.dtype.  Scores and softmax are computed in
    ``math_dtype`` (fp32): a straightforward definition, not SDPA's blocked one.
    """
    B, Tn, H, D = q.shape
    Hkv = k_cache.shape[2]
    group = H // Hkv
    out = torch.empty_like(q)
    seqlens = [int(s) for s in cache_seqlens.tolist()]
    scale = 1.0 / math.sqrt(D)
    for b in range(B):
        pos = seqlens[b]
        if k is not None:
            k_cache[b, pos:pos + Tn] = k[b]
            v_cache[b, pos:pos + Tn] = v[b]
        for t in range(Tn):
            lo, hi = key_range(pos, t, window_size[0])
            kk = k_cache[b, lo:hi + 1].to(math_dtype)      # [n,Hkv,D]
            vv = v_cache[b, lo:hi + 1].to(math_dtype)
            kk = kk.repeat_interleave(group, dim=1)        # q head h <-> kv head h // group
            vv = vv.repeat_interleave(group, dim=1)
            qq = q[b, t].to(math_dtype)                    # [H,D]
            s = torch.einsum("hd,nhd->hn", qq, kk) * scale
            p = torch.softmax(s, dim=-1)
            out[b, t] = torch.einsum("hn,nhd->hd", p, vv).to(q.dtype)
    return out


def attention_with_kvcache_sdpa(q, k_cache, v_cache, k=None, v=None, cache_seqlens=None,
                                window_size=(-1, 0)):
    """The reference's CPU behaviour, op for op (uniform position = row 0's),
    built on ``F.scaled_dot_product_attention`` (flash_attention.py:163-185)."""
    B, Tn, H, D = q.shape
    pos = int(cache_seqlens[0].item())
    if k is not None:
        k_cache[:, pos:pos + Tn] = k
        v_cache[:, pos:pos + Tn] = v
    end = pos + Tn
    qs = q.transpose(1, 2)
    ks = k_cache[:, :end].transpose(1, 2)
    vs = v_cache[:, :end].transpose(1, 2)
    gqa = qs.size(1) != ks.size(1)
    w = window_size[0]
    Tk = end
    if (w < 0 or w >= Tn) and Tn == Tk:
        y = F.scaled_dot_product_attention(qs, ks, vs, is_causal=True, enable_gqa=gqa)
    elif Tn == 1:
        if 0 <= w < Tk:
            start = max(0, Tk - (w + 1))
            ks, vs = ks[:, :, start:], vs[:, :, start:]
        y = F.scaled_dot_product_attention(qs, ks, vs, is_causal=False, enable_gqa=gqa)
    else:
        rows = (Tk - Tn) + torch.arange(Tn).unsqueeze(1)
        cols = torch.arange(Tk).unsqueeze(0)
        mask = cols <= rows
        if 0 <= w < Tk:
            mask = mask & ((rows - cols) <= w)
        y = F.scaled_dot_product_attention(qs, ks, vs, attn_mask=mask, enable_gqa=gqa)
    return y.transpose(1, 2)
