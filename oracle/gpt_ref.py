"""Oracle: functional GPT forward over a reference-named parameter dict (torch CPU).

Test infrastructure only; never imported by the product package.

Parameter names are the reference's state-dict keys
(``transformer.wte.weight``, ``transformer.h.{i}.attn.c_q.weight``, ...,
``lm_head.weight``, ``resid_lambdas``, ``x0_lambdas``, ``smear_gate.weight``,
``smear_lambda``, ``backout_lambda``, ``value_embeds.{i}.weight``), so a reference
checkpoint's ``model_*.pt`` loads into this oracle unchanged.

Follows nanochat/gpt.py: config :28-39, norm :42-43, has_ve :53-55, rotary :57-65
and :270-285, attention :84-128, MLP :137-141, block :150-153, init :204-268,
windows :287-314, forward :459-524.  Every elementwise step is issued as its own
torch op in the compute dtype, so bf16 rounding happens exactly where the
reference's eager graph rounds.
"""
from dataclasses import dataclass
import math

import torch
import torch.nn.functional as F

from . import fp8_ref
from .attention_ref import attention_with_kvcache, attention_with_kvcache_sdpa

SOFTCAP = 15.0            # gpt.py:511
ROPE_BASE = 100000.0      # gpt.py:270
QK_GAIN = 1.2             # gpt.py:103-104
SMEAR_CHANNELS = 24       # gpt.py:177
VE_GATE_CHANNELS = 12     # gpt.py:81


@dataclass
class GPTConfig:
    sequence_len: int = 2048
    vocab_size: int = 32768
    n_layer: int = 12
    n_head: int = 6
    n_kv_head: int = 6
    n_embd: int = 768
    window_pattern: str = "SSSL"


def has_ve(i, n_layer):
    return i % 2 == (n_layer - 1) % 2


def padded_vocab(cfg, multiple=64):
    return -(-cfg.vocab_size // multiple) * multiple


def window_sizes(cfg):
    """Per-layer (left, right).  S = ceil(seq/4/128)*128 (512 for 2048), L = seq;
    pattern tiled over layers, last layer forced to L (gpt.py:287-314)."""
    long_w = cfg.sequence_len
    short_w = -(-long_w // 4 // 128) * 128
    pat = cfg.window_pattern.upper()
    assert pat and all(c in "SL" for c in pat)
    out = [(long_w if pat[i % len(pat)] == "L" else short_w, 0) for i in range(cfg.n_layer)]
    out[-1] = (long_w, 0)
    return out


def rotary_tables(seq_len, head_dim, dtype, base=ROPE_BASE):
    """cos/sin of t * base^(-2j/D), fp32 then rounded to ``dtype``; [seq, D/2]."""
    j = torch.arange(0, head_dim, 2, dtype=torch.float32)
    inv_freq = 1.0 / (base ** (j / head_dim))
    t = torch.arange(seq_len, dtype=torch.float32)
    ang = torch.outer(t, inv_freq)
    return ang.cos().to(dtype), ang.sin().to(dtype)


def init_params(cfg, seed=0, compute_dtype=torch.float32, trained_like=False, master_dtype=torch.float32):
    """Random init in the reference's RNG call order (gpt.py:220-255).

    ``trained_like`` replaces the zero-initialised projections and zero smear
    lambda by small random values (drawn afterwards, so the first part of the
    stream is unchanged) so that attention, MLP, smear and the KV cache all
    influence the logits.
    """
    torch.manual_seed(seed)
    E, L = cfg.n_embd, cfg.n_layer
    D = E // cfg.n_head
    kv_dim = cfg.n_kv_head * D
    V = padded_vocab(cfg)
    p = {}
    p["transformer.wte.weight"] = torch.empty(V, E).normal_(0.0, 0.8)
    p["lm_head.weight"] = torch.empty(V, E).normal_(0.0, 0.001)
    s = 3 ** 0.5 * E ** -0.5
    for i in range(L):
        pre = f"transformer.h.{i}."
        p[pre + "attn.c_q.weight"] = torch.empty(cfg.n_head * D, E).uniform_(-s, s)
        p[pre + "attn.c_k.weight"] = torch.empty(kv_dim, E).uniform_(-s, s)
        p[pre + "attn.c_v.weight"] = torch.empty(kv_dim, E).uniform_(-s, s)
        p[pre + "attn.c_proj.weight"] = torch.zeros(E, E)
        p[pre + "mlp.c_fc.weight"] = torch.empty(4 * E, E).uniform_(-s * 0.4, s * 0.4)
        p[pre + "mlp.c_proj.weight"] = torch.zeros(E, 4 * E)
    p["resid_lambdas"] = torch.tensor([1.15 - 0.10 * i / max(L - 1, 1) for i in range(L)])
    p["x0_lambdas"] = torch.tensor([0.20 - 0.15 * i / max(L - 1, 1) for i in range(L)])
    p["smear_lambda"] = torch.zeros(1)
    p["backout_lambda"] = torch.full((1,), 0.2)
    p["smear_gate.weight"] = torch.empty(1, SMEAR_CHANNELS).uniform_(0.0, 0.02)
    for i in range(L):
        if has_ve(i, L):
            p[f"value_embeds.{i}.weight"] = torch.empty(V, kv_dim).uniform_(-s, s)
    for i in range(L):
        if has_ve(i, L):
            p[f"transformer.h.{i}.attn.ve_gate.weight"] = torch.empty(cfg.n_kv_head, VE_GATE_CHANNELS).uniform_(0.0, 0.02)
    if trained_like:
        for i in range(L):
            pre = f"transformer.h.{i}."
            p[pre + "attn.c_proj.weight"].uniform_(-s, s)
            p[pre + "mlp.c_proj.weight"].uniform_(-s * 0.5, s * 0.5)
        p["smear_lambda"].fill_(0.35)
        p["smear_gate.weight"].uniform_(-0.5, 0.5)
        p["lm_head.weight"].normal_(0.0, 0.03)
        for i in range(L):
            if has_ve(i, L):
                p[f"transformer.h.{i}.attn.ve_gate.weight"].uniform_(-0.5, 0.5)
    if compute_dtype != torch.float16:                      # gpt.py:264-267
        p["transformer.wte.weight"] = p["transformer.wte.weight"].to(compute_dtype)
        for i in range(L):
            if has_ve(i, L):
                p[f"value_embeds.{i}.weight"] = p[f"value_embeds.{i}.weight"].to(compute_dtype)
    if master_dtype != torch.float32:
        for k_ in list(p):
            if p[k_].dtype == torch.float32 and p[k_].ndim == 2:
                p[k_] = p[k_].to(master_dtype)
    return p


def rms_norm(x):
    return F.rms_norm(x, (x.size(-1),))


def small_linear(x, w):
    """The reference's cast-on-the-fly Linear (gpt.py:45-50)."""
    return F.linear(x, w.to(x.dtype))


def rotate(x, cos, sin):
    """Half-split rotation by -theta (gpt.py:57-65). x [B,T,H,D]; cos/sin [1,T,1,D/2]."""
    d = x.shape[-1] // 2
    x1, x2 = x[..., :d], x[..., d:]
    y1 = x1 * cos + x2 * sin
    y2 = x1 * (-sin) + x2 * cos
    return torch.cat([y1, y2], dim=-1)


class Runtime:
    """Per-model oracle state: config, params, tables, linear flavour."""

    def __init__(self, cfg, params, compute_dtype=torch.bfloat16, fp8=True,
                 cache_weights=True, uniform_sdpa=True):
        self.cfg = cfg
        self.p = params
        self.dtype = compute_dtype
        self.fp8 = fp8
        self.wcache = fp8_ref.WeightCache() if cache_weights else None
        self.uniform_sdpa = uniform_sdpa
        D = cfg.n_embd // cfg.n_head
        cos, sin = rotary_tables(cfg.sequence_len * 10, D, compute_dtype)
        self.cos = cos[None, :, None, :]
        self.sin = sin[None, :, None, :]
        self.windows = window_sizes(cfg)
        self.taps = None      # optional dict filled with intermediate tensors

    def linear(self, x, name):
        w = self.p[name]
        out_f, in_f = w.shape
        if self.fp8 and fp8_ref.fp8_module_filter(in_f, out_f):
            return fp8_ref.float8_linear(x, w, compute_dtype=self.dtype, wcache=self.wcache)
        return small_linear(x, w)

    def tap(self, key, value):
        if self.taps is not None:
            self.taps[key] = value.detach().clone()


@torch.no_grad()
def forward(rt: Runtime, idx, kv_cache=None):
    """GPT.forward(idx, kv_cache=...) -> fp32 logits [B,T,vocab] (gpt.py:459-524).

    With ``kv_cache=None`` the whole sequence is attended causally with no cache
    (the reference's training-style forward, T > 1)."""
    cfg, p, dt = rt.cfg, rt.p, rt.dtype
    B, T = idx.shape
    H, Hkv = cfg.n_head, cfg.n_kv_head
    D = cfg.n_embd // H
    L = cfg.n_layer
    if kv_cache is None:
        T0 = 0
    elif rt.uniform_sdpa:
        T0 = kv_cache.get_pos()
    else:
        T0 = None
    if T0 is not None:
        cos, sin = rt.cos[:, T0:T0 + T], rt.sin[:, T0:T0 + T]
    else:  # ragged rows: per-row positions
        posv = kv_cache.cache_seqlens.long()[:, None] + torch.arange(T)[None, :]   # [B,T]
        cos, sin = rt.cos[0, posv], rt.sin[0, posv]                                 # [B,T,1,D/2]

    x = F.embedding(idx, p["transformer.wte.weight"]).to(dt)
    x = rms_norm(x)
    lam_s = p["smear_lambda"].to(x.dtype)
    gate_w = p["smear_gate.weight"]
    if kv_cache is None:
        assert T > 1
        gate = lam_s * torch.sigmoid(small_linear(x[:, 1:, :SMEAR_CHANNELS], gate_w))
        x = torch.cat([x[:, :1], x[:, 1:] + gate * x[:, :-1]], dim=1)
    else:
        prev = kv_cache.prev_embedding
        kv_cache.prev_embedding = x[:, -1:, :]
        if T > 1:
            gate = lam_s * torch.sigmoid(small_linear(x[:, 1:, :SMEAR_CHANNELS], gate_w))
            x = torch.cat([x[:, :1], x[:, 1:] + gate * x[:, :-1]], dim=1)
        elif prev is not None:
            gate = lam_s * torch.sigmoid(small_linear(x[:, :, :SMEAR_CHANNELS], gate_w))
            x = x + gate * prev
    rt.tap("xemb", x)

    x0 = x
    x_backout = None
    for i in range(L):
        pre = f"transformer.h.{i}."
        x = p["resid_lambdas"][i] * x + p["x0_lambdas"][i] * x0
        rt.tap(f"xmix{i}", x)
        ve_name = f"value_embeds.{i}.weight"
        ve = F.embedding(idx, p[ve_name]).to(x.dtype) if ve_name in p else None
        # --- attention
        xn = rms_norm(x)
        rt.tap(f"xn{i}", xn)
        q = rt.linear(xn, pre + "attn.c_q.weight").view(B, T, H, D)
        k = rt.linear(xn, pre + "attn.c_k.weight").view(B, T, Hkv, D)
        v = rt.linear(xn, pre + "attn.c_v.weight").view(B, T, Hkv, D)
        if rt.taps is not None:
            rt.tap(f"qkv{i}", torch.cat([q.reshape(B, T, -1), k.reshape(B, T, -1), v.reshape(B, T, -1)], dim=-1))
        if ve is not None:
            ve = ve.view(B, T, Hkv, D)
            g = 3 * torch.sigmoid(small_linear(xn[..., :VE_GATE_CHANNELS], p[pre + "attn.ve_gate.weight"]))
            v = v + g.unsqueeze(-1) * ve
        q, k = rotate(q, cos, sin), rotate(k, cos, sin)
        q, k = rms_norm(q), rms_norm(k)
        q = q * QK_GAIN
        k = k * QK_GAIN
        rt.tap(f"q{i}", q)
        w = rt.windows[i]
        if kv_cache is None:
            kc = torch.zeros(B, T, Hkv, D, dtype=dt)
            vc = torch.zeros(B, T, Hkv, D, dtype=dt)
            zeros = torch.zeros(B, dtype=torch.int32)
            y = attention_with_kvcache_sdpa(q, kc, vc, k, v, zeros, w)
        else:
            kc, vc = kv_cache.get_layer_cache(i)
            if rt.uniform_sdpa:
                y = attention_with_kvcache_sdpa(q, kc, vc, k, v, kv_cache.cache_seqlens, w)
            else:
                y = attention_with_kvcache(q, kc, vc, k, v, kv_cache.cache_seqlens, w)
            if i == kv_cache.n_layers - 1:
                kv_cache.advance(T)
        rt.tap(f"y{i}", y)
        y = y.contiguous().view(B, T, -1)
        attn_out = rt.linear(y, pre + "attn.c_proj.weight")
        rt.tap(f"attn_out{i}", attn_out)
        x = x + attn_out
        rt.tap(f"xmid{i}", x)
        # --- MLP
        xn2 = rms_norm(x)
        rt.tap(f"xn2_{i}", xn2)
        h = rt.linear(xn2, pre + "mlp.c_fc.weight")
        h = F.relu(h).square()
        rt.tap(f"h2_{i}", h)
        mlp_out = rt.linear(h, pre + "mlp.c_proj.weight")
        rt.tap(f"mlp_out{i}", mlp_out)
        x = x + mlp_out
        rt.tap(f"x{i}", x)
        if i == L // 2:
            x_backout = x
    if x_backout is not None:
        x = x - p["backout_lambda"].to(x.dtype) * x_backout
    x = rms_norm(x)
    rt.tap("xf", x)
    logits = rt.linear(x, "lm_head.weight")
    logits = logits[..., :cfg.vocab_size].float()
    logits = SOFTCAP * torch.tanh(logits / SOFTCAP)
    return logits


# ---- cost accounting (gpt.py:341-388, scripts/infer_bench.py:51-53) -------------------

def kv_bytes_per_token(cfg, itemsize=2):
    D = cfg.n_embd // cfg.n_head
    return cfg.n_layer * 2 * cfg.n_kv_head * D * itemsize


def kv_read_bytes(cfg, context_len, itemsize=2):
    D = cfg.n_embd // cfg.n_head
    return sum(2 * cfg.n_kv_head * D * itemsize * min(context_len, w) for w, _ in window_sizes(cfg))


def num_matmul_params(params):
    """All weights that multiply the token stream (every 2-D weight that is not an
    embedding table), counting FP8-converted layers too."""
    return sum(v.numel() for k, v in params.items()
               if v.ndim == 2 and "wte" not in k and "value_embeds" not in k)


def estimate_decode_flops(cfg, params, context_len):
    D = cfg.n_embd // cfg.n_head
    attn = sum(4 * cfg.n_head * D * min(context_len, w) for w, _ in window_sizes(cfg))
    return 2 * num_matmul_params(params) + attn
