"""Pins the attention / GPT / sampler oracle (CPU only).

  * attention: brute-force softmax vs SDPA form, window = last w+1 keys, GQA = repeat_interleave,
    single key => output = v, in-place append (the behaviours the reference's
    tests/test_attention_fallback.py pins)
  * rms-norm / rotary closed forms and invariants
  * GPT: golden greedy ids + logits written by the reference's own GPT on the seeded d4 model
    (fp32 and bf16+FP8), weight hashes, cached decode == cache-free forward
  * sampler: multinomial identity, argmax first index
"""
import hashlib
import json
import math
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import gpt_ref, decode_ref
from oracle.attention_ref import attention_with_kvcache, attention_with_kvcache_sdpa, key_range

GOLD_DIR = os.path.join(os.path.dirname(__file__), "golden")


def sha(t):
    t = t.detach().contiguous()
    raw = t.view(torch.int16).numpy().tobytes() if t.dtype == torch.bfloat16 else t.numpy().tobytes()
    return hashlib.sha256(raw).hexdigest()


# ------------------------------------------------------------------ attention
def brute_attention(q, K, V):
    """q [D], K,V [n,D] python-float softmax."""
    D = q.numel()
    s = [sum(float(q[d]) * float(K[j, d]) for d in range(D)) / math.sqrt(D) for j in range(K.shape[0])]
    m = max(s)
    e = [math.exp(v - m) for v in s]
    z = sum(e)
    return [sum(e[j] / z * float(V[j, d]) for j in range(K.shape[0])) for d in range(D)]


def test_attention_bruteforce_window_gqa():
    g = torch.Generator().manual_seed(0)
    B, Tmax, H, Hkv, D = 2, 12, 4, 2, 8
    kc = torch.randn(B, Tmax, Hkv, D, generator=g)
    vc = torch.randn(B, Tmax, Hkv, D, generator=g)
    q = torch.randn(B, 1, H, D, generator=g)
    k = torch.randn(B, 1, Hkv, D, generator=g)
    v = torch.randn(B, 1, Hkv, D, generator=g)
    seq = torch.tensor([7, 3], dtype=torch.int32)
    w = 4
    out = attention_with_kvcache(q, kc, vc, k, v, seq, (w, 0))
    for b in range(B):
        pos = int(seq[b])
        assert torch.equal(kc[b, pos], k[b, 0]) and torch.equal(vc[b, pos], v[b, 0])   # appended in place
        lo, hi = key_range(pos, 0, w)
        assert hi - lo + 1 == min(pos + 1, w + 1)
        for h in range(H):
            want = brute_attention(q[b, 0, h], kc[b, lo:hi + 1, h // 2], vc[b, lo:hi + 1, h // 2])
            assert torch.allclose(out[b, 0, h], torch.tensor(want), atol=1e-5)


def test_attention_single_key_is_v_and_sdpa_agreement():
    g = torch.Generator().manual_seed(1)
    B, Tmax, H, D = 2, 40, 4, 16
    kc = torch.zeros(B, Tmax, H, D)
    vc = torch.zeros(B, Tmax, H, D)
    q = torch.randn(B, 1, H, D, generator=g)
    k = torch.randn(B, 1, H, D, generator=g)
    v = torch.randn(B, 1, H, D, generator=g)
    out = attention_with_kvcache(q, kc, vc, k, v, torch.zeros(B, dtype=torch.int32), (Tmax, 0))
    assert torch.allclose(out, v, atol=1e-6)
    # prefill of 16 then decode with a window smaller than the cache (the reference's sliding-window case)
    kc.zero_(), vc.zero_()
    kc2, vc2 = kc.clone(), vc.clone()
    qp, kp, vp = (torch.randn(B, 33, H, D, generator=g) for _ in range(3))
    zero = torch.zeros(B, dtype=torch.int32)
    a = attention_with_kvcache(qp, kc, vc, kp, vp, zero, (8, 0))
    b = attention_with_kvcache_sdpa(qp, kc2, vc2, kp, vp, zero, (8, 0))
    assert torch.allclose(a, b, atol=1e-5) and torch.equal(kc, kc2)
    seq = torch.full((B,), 33, dtype=torch.int32)
    a = attention_with_kvcache(q, kc, vc, k, v, seq, (8, 0))
    b = attention_with_kvcache_sdpa(q, kc2, vc2, k, v, seq, (8, 0))
    assert torch.allclose(a, b, atol=1e-5)
    # GQA == repeat_interleave of kv heads
    kc3 = torch.randn(B, 10, 2, D, generator=g)
    vc3 = torch.randn(B, 10, 2, D, generator=g)
    seq = torch.full((B,), 10, dtype=torch.int32)
    a = attention_with_kvcache(q, kc3, vc3, None, None, seq - 1, (-1, 0))
    b = attention_with_kvcache(q, kc3.repeat_interleave(2, 2), vc3.repeat_interleave(2, 2), None, None, seq - 1, (-1, 0))
    assert torch.allclose(a, b, atol=1e-6)


# ------------------------------------------------------------------ norm / rotary
def test_rms_norm_and_rotary_closed_forms():
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 128, generator=g)
    y = gpt_ref.rms_norm(x)
    assert torch.allclose(y.pow(2).mean(-1), torch.ones(3), atol=1e-5)
    assert torch.allclose(gpt_ref.rms_norm(7.5 * x), y, atol=1e-5)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 2.0 ** -23)
    assert torch.allclose(y, want, atol=1e-6)
    cos, sin = gpt_ref.rotary_tables(64, 128, torch.float32)
    assert cos.shape == (64, 64) and torch.all(cos[0] == 1) and torch.all(sin[0] == 0)
    assert abs(cos[5, 3].item() - math.cos(5 * 100000.0 ** (-6 / 128))) < 1e-6
    q = torch.randn(1, 64, 2, 128, generator=g)
    k = torch.randn(1, 64, 2, 128, generator=g)
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    rq, rk = gpt_ref.rotate(q, c, s), gpt_ref.rotate(k, c, s)
    assert torch.equal(rq[:, 0], q[:, 0])                                   # position 0 is the identity
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1), atol=1e-4)       # rotation preserves norms
    # <rot(q,m), rot(k,n)> depends on m-n only
    qq = q[:, :1].expand(-1, 64, -1, -1)
    kk = k[:, :1].expand(-1, 64, -1, -1)
    rq, rk = gpt_ref.rotate(qq, c, s), gpt_ref.rotate(kk, c, s)
    d1 = (rq[0, 10, 0] * rk[0, 4, 0]).sum()
    d2 = (rq[0, 36, 0] * rk[0, 30, 0]).sum()
    assert abs(d1 - d2) < 1e-3
    # y1 = x1 cos + x2 sin ; y2 = -x1 sin + x2 cos  (rotation by -theta)
    x1, x2 = q[0, 7, 0, :64], q[0, 7, 0, 64:]
    r = gpt_ref.rotate(q, c, s)[0, 7, 0]
    assert torch.allclose(r[:64], x1 * cos[7] + x2 * sin[7], atol=1e-6)
    assert torch.allclose(r[64:], -x1 * sin[7] + x2 * cos[7], atol=1e-6)


def test_window_sizes_and_value_embed_layers():
    cfg = gpt_ref.GPTConfig(n_layer=26, n_head=13, n_kv_head=13, n_embd=1664)
    w = gpt_ref.window_sizes(cfg)
    assert [i for i, (x, _) in enumerate(w) if x == 2048] == [3, 7, 11, 15, 19, 23, 25]
    assert all(x in (512, 2048) for x, _ in w)
    assert [i for i in range(26) if gpt_ref.has_ve(i, 26)] == list(range(1, 26, 2))
    assert gpt_ref.kv_read_bytes(cfg, 2048) == 64 * 0 + (7 * 2048 + 19 * 512) * 2 * 13 * 128 * 2
    assert gpt_ref.kv_bytes_per_token(cfg) == 26 * 2 * 13 * 128 * 2


# ------------------------------------------------------------------ GPT vs the reference's goldens
def load_gold(name):
    with open(os.path.join(GOLD_DIR, name)) as f:
        return json.load(f)


def check_digest(row, dig, atol):
    assert torch.allclose(row[:32], torch.tensor(dig["head"]), atol=atol, rtol=0)
    assert torch.allclose(row[::1021], torch.tensor(dig["strided"]), atol=atol, rtol=0)
    assert torch.allclose(row[dig["top_idx"]], torch.tensor(dig["top_val"]), atol=atol, rtol=0)


@pytest.mark.parametrize("gold_name,dtype,fp8", [("gpt_d4_fp32.json", torch.float32, False),
                                                 ("gpt_d4_bf16_fp8.json", torch.bfloat16, True)])
@pytest.mark.parametrize("init", ["repo", "trained_like"])
def test_gpt_oracle_matches_reference_goldens(gold_name, dtype, fp8, init):
    gold = load_gold(gold_name)
    cfg = gpt_ref.GPTConfig(**gold["config"])
    params = gpt_ref.init_params(cfg, seed=0, compute_dtype=dtype, trained_like=(init == "trained_like"))
    run = gold["runs"][init]
    mism = [k for k, h in run["weight_sha256"].items() if sha(params[k]) != h]
    if mism:
        pytest.skip(f"this host's torch RNG does not reproduce the golden weights ({mism[:3]} ...)")
    rt = gpt_ref.Runtime(cfg, params, compute_dtype=dtype, fp8=fp8)
    n = 24
    toks, logits = decode_ref.generate(rt, gold["prompt"], 1, n, temperature=0.0, collect_logits=True)
    # The oracle follows the same op sequence, so on the same host it reproduces the reference bit for bit.
    atol = 0.0
    for t in range(n):
        check_digest(logits[t][0], run["steps"][t]["digest"], atol)
    assert [c[0] for c in toks] == run["greedy_ids"][:n]


def test_cached_decode_equals_cache_free_forward():
    gold = load_gold("gpt_d4_fp32.json")
    cfg = gpt_ref.GPTConfig(**gold["config"])
    params = gpt_ref.init_params(cfg, seed=0, compute_dtype=torch.float32, trained_like=True)
    rt = gpt_ref.Runtime(cfg, params, compute_dtype=torch.float32, fp8=False)
    prompt = gold["prompt"][:12]
    a, _ = decode_ref.generate(rt, prompt, 1, 6, temperature=0.0)
    b = decode_ref.generate_nocache(rt, prompt, 6)
    assert [c[0] for c in a] == b
    ref = gold["runs"]["repo"]
    if "nocache_ids" in ref:   # the reference's own cache-free ids equal its cached ids
        assert ref["nocache_ids"] == ref["greedy_ids"][:len(ref["nocache_ids"])]


def test_ragged_rows_equal_row_by_row():
    cfg = gpt_ref.GPTConfig(sequence_len=64, vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=64)
    params = gpt_ref.init_params(cfg, seed=3, compute_dtype=torch.float32, trained_like=True)
    g = torch.Generator().manual_seed(0)
    lens = [5, 9]
    prompts = [torch.randint(0, 256, (n,), generator=g).tolist() for n in lens]
    nxt = torch.randint(0, 256, (2, 1), generator=g)
    rows = []
    rt1 = gpt_ref.Runtime(cfg, params, compute_dtype=torch.float32, fp8=False)
    caches = []
    for pr in prompts:
        c = decode_ref.new_cache(cfg, 1, 16, torch.float32)
        gpt_ref.forward(rt1, torch.tensor([pr]), c)
        caches.append(c)
    for b in range(2):
        rows.append(gpt_ref.forward(rt1, nxt[b:b + 1], caches[b])[0, -1])
    # same thing as one ragged batch
    rt2 = gpt_ref.Runtime(cfg, params, compute_dtype=torch.float32, fp8=False, uniform_sdpa=False)
    big = decode_ref.new_cache(cfg, 2, 16, torch.float32)
    for b in range(2):
        c = decode_ref.new_cache(cfg, 1, 16, torch.float32)
        gpt_ref.forward(rt1, torch.tensor([prompts[b]]), c)
        big.k_cache[:, b] = c.k_cache[:, 0]
        big.v_cache[:, b] = c.v_cache[:, 0]
        big.cache_seqlens[b] = lens[b]
        prev = c.prev_embedding if b == 0 else torch.cat([prev, c.prev_embedding], 0)
    big.prev_embedding = prev
    out = gpt_ref.forward(rt2, nxt, big)[:, -1]
    assert torch.allclose(out, torch.stack(rows), atol=2e-5)


# ------------------------------------------------------------------ sampler
def test_sampler_identities():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(6, 300, generator=g) * 3
    assert torch.equal(decode_ref.sample_next_token(logits, None, 0.0), logits.argmax(-1, keepdim=True))
    tie = torch.zeros(2, 50)
    assert decode_ref.sample_next_token(tie, None, 0.0).flatten().tolist() == [0, 0]
    for temp, k in [(1.0, 50), (0.6, 7), (1.3, None)]:
        r1 = torch.Generator().manual_seed(11)
        r2 = torch.Generator().manual_seed(11)
        want = decode_ref.sample_next_token(logits, r1, temp, k)
        width = min(k, 300) if k else 300
        noise = torch.empty(6, width).exponential_(1.0, generator=r2)
        got = decode_ref.sample_with_noise(logits, temp, k, noise)
        assert torch.equal(want, got)
