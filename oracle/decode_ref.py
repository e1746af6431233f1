"""Oracle: KV-cache container, next-token sampler and a minimal generate loop.

Test infrastructure only; never imported by the product package.

Follows nanochat/engine.py: KVCache :82-137, sample_next_token :140-156 and the
prefill -> replicate -> sample/forward loop of Engine.generate :194-275 (without
the tool-use state machine, which is host-only logic tested on the product class).
"""
import torch
import torch.nn.functional as F

from . import gpt_ref


class RefKVCache:
    def __init__(self, batch_size, num_heads, seq_len, head_dim, num_layers, dtype=torch.float32):
        self.batch_size, self.max_seq_len = batch_size, seq_len
        self.n_layers, self.n_heads, self.head_dim = num_layers, num_heads, head_dim
        shape = (num_layers, batch_size, seq_len, num_heads, head_dim)
        self.k_cache = torch.zeros(shape, dtype=dtype)
        self.v_cache = torch.zeros(shape, dtype=dtype)
        self.cache_seqlens = torch.zeros(batch_size, dtype=torch.int32)
        self.prev_embedding = None

    def get_pos(self):
        return int(self.cache_seqlens[0].item())

    def get_layer_cache(self, i):
        return self.k_cache[i], self.v_cache[i]

    def advance(self, n):
        self.cache_seqlens += n

    def prefill(self, other):
        assert self.get_pos() == 0
        assert (self.n_layers, self.n_heads, self.head_dim) == (other.n_layers, other.n_heads, other.head_dim)
        assert self.max_seq_len >= other.max_seq_len
        n = other.get_pos()
        self.k_cache[:, :, :n] = other.k_cache[:, :, :n]
        self.v_cache[:, :, :n] = other.v_cache[:, :, :n]
        self.cache_seqlens.fill_(n)
        if other.prev_embedding is not None:
            self.prev_embedding = other.prev_embedding.expand(self.batch_size, -1, -1).clone()


def new_cache(cfg, batch, seq_len, dtype):
    return RefKVCache(batch, cfg.n_kv_head, seq_len, cfg.n_embd // cfg.n_head, cfg.n_layer, dtype)


def sample_with_noise(logits, temperature, top_k, noise):
    """engine.py:140-156 with torch.multinomial written out as its definition:
    multinomial(p, 1) == argmax(p / e), e ~ Exp(1) drawn from the generator.
    ``noise`` holds those exponentials, shape [B, k] (or [B, V] without top-k).

    torch.topk leaves the order of equal values unspecified (it differs between its CPU and GPU kernels), and bf16-rounded
    logits tie often; equal values are taken lowest index first here (a stable descending sort), which is one of the
    orders torch.topk may return and equals it whenever the k+1 largest values are distinct."""
    if temperature == 0.0:
        return torch.argmax(logits, dim=-1, keepdim=True)
    if top_k is not None and top_k > 0:
        k = min(top_k, logits.size(-1))
        vals, idx = torch.sort(logits, dim=-1, descending=True, stable=True)
        vals, idx = vals[:, :k], idx[:, :k]
        probs = F.softmax(vals / temperature, dim=-1)
        choice = torch.argmax(probs / noise, dim=-1, keepdim=True)
        return idx.gather(1, choice)
    probs = F.softmax(logits / temperature, dim=-1)
    return torch.argmax(probs / noise, dim=-1, keepdim=True)


def sample_next_token(logits, rng, temperature=1.0, top_k=None):
    """The reference's sampler verbatim in behaviour (engine.py:140-156)."""
    assert temperature >= 0.0
    if temperature == 0.0:
        return torch.argmax(logits, dim=-1, keepdim=True)
    if top_k is not None and top_k > 0:
        k = min(top_k, logits.size(-1))
        vals, idx = torch.topk(logits, k, dim=-1)
        probs = F.softmax(vals / temperature, dim=-1)
        return idx.gather(1, torch.multinomial(probs, 1, generator=rng))
    return torch.multinomial(F.softmax(logits / temperature, dim=-1), 1, generator=rng)


@torch.no_grad()
def generate(rt, prompt, num_samples=1, max_tokens=16, temperature=0.0, top_k=None, seed=42,
             collect_logits=False):
    """Prefill at B=1, replicate the cache, then decode (engine.py:194-275).

    Returns (tokens [max_tokens][num_samples], logits list or None)."""
    cfg = rt.cfg
    rng = torch.Generator().manual_seed(seed)
    pre = new_cache(cfg, 1, len(prompt), rt.dtype)
    ids = torch.tensor([prompt], dtype=torch.long)
    logits = gpt_ref.forward(rt, ids, pre)[:, -1, :].expand(num_samples, -1)
    dec = new_cache(cfg, num_samples, len(prompt) + max_tokens, rt.dtype)
    dec.prefill(pre)
    out, kept = [], []
    for step in range(max_tokens):
        if collect_logits:
            kept.append(logits.clone())
        nxt = sample_next_token(logits, rng, temperature, top_k)
        col = nxt[:, 0].tolist()
        out.append(col)
        if step == max_tokens - 1:
            break   # the reference runs one more (unused) forward here; skipped
        ids = torch.tensor(col, dtype=torch.long).unsqueeze(1)
        logits = gpt_ref.forward(rt, ids, dec)[:, -1, :]
    return out, (kept if collect_logits else None)


@torch.no_grad()
def generate_nocache(rt, prompt, max_tokens):
    """Greedy full-recompute decode (gpt.py:526-555): the cache-free invariant."""
    ids = torch.tensor([prompt], dtype=torch.long)
    out = []
    for _ in range(max_tokens):
        logits = gpt_ref.forward(rt, ids, None)[:, -1, :]
        nxt = torch.argmax(logits, dim=-1, keepdim=True)
        ids = torch.cat([ids, nxt], dim=1)
        out.append(int(nxt.item()))
    return out
