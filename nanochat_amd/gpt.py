"""GPT with the reference's module tree and state-dict keys (nanochat/gpt.py:28-39, 67-201), whose
forward with a KV cache runs as one native call into libnanochat_amd.so.

Scope: inference.  `forward(idx, kv_cache=...)` (decode and prefill) and the cache-free
`forward(idx)` are implemented on the GPU; `targets=` (training loss) is not part of this path and
raises.  All six linears of every block and lm_head must be Float8Linear (convert_to_float8_training
with fp8_module_filter): their weights are quantized once into a packed plan (q|k|v stacked into one
weight with three scales) that is rebuilt whenever a weight changes.
"""
import ctypes as C
from dataclasses import dataclass

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import _lib, ops
from .common import COMPUTE_DTYPE
from .fp8 import Float8Linear


@dataclass
class GPTConfig:
    sequence_len: int = 2048
    vocab_size: int = 32768
    n_layer: int = 12
    n_head: int = 6
    n_kv_head: int = 6
    n_embd: int = 768
    window_pattern: str = "SSSL"


def has_ve(layer_idx, n_layer):
    """Value embeddings sit on alternating layers, the last one included (gpt.py:53-55)."""
    return layer_idx % 2 == (n_layer - 1) % 2


class Linear(nn.Linear):
    """Linear whose weight is cast to the input's dtype in forward (gpt.py:45-50): master weights stay fp32, the product runs in
    the activation dtype.  Only the tiny gates (ve_gate [n_kv_head, 12], smear_gate [1, 24]) stay in this class once the FP8
    filter has run, and GPT.forward evaluates those inside its fused kernels; this forward serves a direct call on the module."""

    def forward(self, x):
        return F.linear(x, self.weight.to(dtype=x.dtype))


class CausalSelfAttention(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        self.layer_idx = layer_idx
        self.n_head, self.n_kv_head, self.n_embd = config.n_head, config.n_kv_head, config.n_embd
        self.head_dim = self.n_embd // self.n_head
        assert self.n_embd % self.n_head == 0
        assert self.n_kv_head <= self.n_head and self.n_head % self.n_kv_head == 0
        self.c_q = Linear(self.n_embd, self.n_head * self.head_dim, bias=False)
        self.c_k = Linear(self.n_embd, self.n_kv_head * self.head_dim, bias=False)
        self.c_v = Linear(self.n_embd, self.n_kv_head * self.head_dim, bias=False)
        self.c_proj = Linear(self.n_embd, self.n_embd, bias=False)
        self.ve_gate_channels = 12
        self.ve_gate = Linear(self.ve_gate_channels, self.n_kv_head, bias=False) if has_ve(layer_idx, config.n_layer) else None


class MLP(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.c_fc = Linear(config.n_embd, 4 * config.n_embd, bias=False)
        self.c_proj = Linear(4 * config.n_embd, config.n_embd, bias=False)


class Block(nn.Module):
    def __init__(self, config, layer_idx):
        super().__init__()
        self.attn = CausalSelfAttention(config, layer_idx)
        self.mlp = MLP(config)


def compute_window_sizes(config):
    """(left, right) per layer: S = ceil(seq/4/128)*128, L = seq, last layer L (gpt.py:287-314)."""
    pattern = config.window_pattern.upper()
    assert all(c in "SL" for c in pattern), f"Invalid window_pattern: {pattern}. Use only S and L."
    long_w = config.sequence_len
    short_w = -(-long_w // 4 // 128) * 128
    sizes = [((long_w if pattern[i % len(pattern)] == "L" else short_w), 0) for i in range(config.n_layer)]
    sizes[-1] = (long_w, 0)
    return sizes


class GPT(nn.Module):
    SOFTCAP = 15.0
    WORKSPACE_CACHE_BYTES = 2 << 30       # step workspaces kept alive between calls (one per (batch, tokens) shape seen)

    def __init__(self, config, pad_vocab_size_to=64):
        super().__init__()
        self.config = config
        self.window_sizes = compute_window_sizes(config)
        padded = -(-config.vocab_size // pad_vocab_size_to) * pad_vocab_size_to
        self.padded_vocab_size = padded
        self.transformer = nn.ModuleDict({
            "wte": nn.Embedding(padded, config.n_embd),
            "h": nn.ModuleList([Block(config, i) for i in range(config.n_layer)]),
        })
        self.lm_head = Linear(config.n_embd, padded, bias=False)
        self.resid_lambdas = nn.Parameter(torch.ones(config.n_layer))
        self.x0_lambdas = nn.Parameter(torch.zeros(config.n_layer))
        self.smear_gate = Linear(24, 1, bias=False)
        self.smear_lambda = nn.Parameter(torch.zeros(1))
        self.backout_lambda = nn.Parameter(0.2 * torch.ones(1))
        head_dim = config.n_embd // config.n_head
        kv_dim = config.n_kv_head * head_dim
        self.value_embeds = nn.ModuleDict({str(i): nn.Embedding(padded, kv_dim)
                                           for i in range(config.n_layer) if has_ve(i, config.n_layer)})
        self.rotary_seq_len = config.sequence_len * 10
        self._plan = None
        self._plan_key = None
        self._plan_params = None
        self._workspaces = {}
        # anything that replaces parameter tensors drops the weight plan (the per-call check below only looks at versions)
        self.register_load_state_dict_post_hook(lambda module, incompatible: module.invalidate_plan())

    # -------------------------------------------------------------------------------------------
    @torch.no_grad()
    def init_weights(self):
        """The reference's initialisation, draw for draw (gpt.py:204-268): the random stream is consumed in the same
        order by the same distributions, so a seeded CPU init gives the reference's weights bit for bit.

        wte normal(0, 0.8); lm_head normal(0, 0.001); per block c_q, c_k, c_v uniform(+-s), attn.c_proj zero,
        c_fc uniform(+-0.4 s), mlp.c_proj zero, with s = sqrt(3 / n_embd); resid / x0 lambdas on linear ramps;
        smear_lambda 0, backout_lambda 0.2, smear_gate uniform(0, 0.02); value embeddings uniform(+-s); value-embedding
        gates uniform(0, 0.02); finally the embedding tables go to the compute dtype (not for fp16)."""
        cfg = self.config
        nn.init.normal_(self.transformer.wte.weight, mean=0.0, std=0.8)
        nn.init.normal_(self.lm_head.weight, mean=0.0, std=0.001)
        s = 3 ** 0.5 * cfg.n_embd ** -0.5
        for block in self.transformer.h:
            nn.init.uniform_(block.attn.c_q.weight, -s, s)
            nn.init.uniform_(block.attn.c_k.weight, -s, s)
            nn.init.uniform_(block.attn.c_v.weight, -s, s)
            nn.init.zeros_(block.attn.c_proj.weight)
            nn.init.uniform_(block.mlp.c_fc.weight, -s * 0.4, s * 0.4)
            nn.init.zeros_(block.mlp.c_proj.weight)
        L = cfg.n_layer
        for i in range(L):
            self.resid_lambdas.data[i] = 1.15 - (0.10 * i / max(L - 1, 1))
            self.x0_lambdas.data[i] = 0.20 - (0.15 * i / max(L - 1, 1))
        nn.init.zeros_(self.smear_lambda)
        nn.init.constant_(self.backout_lambda, 0.2)
        nn.init.uniform_(self.smear_gate.weight, 0.0, 0.02)
        for ve in self.value_embeds.values():
            nn.init.uniform_(ve.weight, -s, s)
        for block in self.transformer.h:
            if block.attn.ve_gate is not None:
                nn.init.uniform_(block.attn.ve_gate.weight, 0.0, 0.02)
        # the rotary tables are rebuilt with the weight plan (rotary_tables), nothing to store here
        if COMPUTE_DTYPE != torch.float16:
            self.transformer.wte.to(dtype=COMPUTE_DTYPE)
            for ve in self.value_embeds.values():
                ve.to(dtype=COMPUTE_DTYPE)
        self.invalidate_plan()

    def get_device(self):
        return self.transformer.wte.weight.device

    def rotary_tables(self, device):
        """bf16 cos/sin of t * 100000^(-2j/D), computed in fp32 (gpt.py:270-285); [seq, D/2]."""
        D = self.config.n_embd // self.config.n_head
        j = torch.arange(0, D, 2, dtype=torch.float32, device=device)
        inv_freq = 1.0 / (100000 ** (j / D))
        t = torch.arange(self.rotary_seq_len, dtype=torch.float32, device=device)
        ang = torch.outer(t, inv_freq)
        return ang.cos().bfloat16().contiguous(), ang.sin().bfloat16().contiguous()

    # ---- cost accounting (gpt.py:341-388); FP8 linears are counted, unlike an isinstance(Linear) test
    def num_matmul_params(self):
        return sum(m.weight.numel() for m in self.modules() if isinstance(m, nn.Linear))

    def estimate_decode_flops(self, context_len):
        h, q = self.config.n_head, self.config.n_embd // self.config.n_head
        attn = sum(4 * h * q * min(context_len, w) for w, _ in self.window_sizes)
        return 2 * self.num_matmul_params() + attn

    def estimate_prefill_flops(self, num_tokens):
        """Causal prefill: token t attends to min(t, window) keys in every layer (gpt.py:362-372)."""
        h, q = self.config.n_head, self.config.n_embd // self.config.n_head
        attn = 0
        for window, _ in self.window_sizes:
            w = min(window, num_tokens)
            attn += 4 * h * q * (w * (w + 1) // 2 + (num_tokens - w) * w)
        return 2 * self.num_matmul_params() * num_tokens + attn

    def kv_bytes_per_token(self):
        D = self.config.n_embd // self.config.n_head
        return self.config.n_layer * 2 * self.config.n_kv_head * D * 2

    def kv_read_bytes(self, context_len):
        D = self.config.n_embd // self.config.n_head
        return sum(2 * self.config.n_kv_head * D * 2 * min(context_len, w) for w, _ in self.window_sizes)

    # -------------------------------------------------------------------------------------------
    def _fp8_modules(self):
        mods = []
        for blk in self.transformer.h:
            mods += [blk.attn.c_q, blk.attn.c_k, blk.attn.c_v, blk.attn.c_proj, blk.mlp.c_fc, blk.mlp.c_proj]
        mods.append(self.lm_head)
        return mods

    def invalidate_plan(self):
        """Forget the quantized-weight plan: the next forward rebuilds it.  Called by everything here that replaces parameter
        tensors (load_state_dict, .to() / .cuda() / dtype casts, the FP8 module swap); call it after assigning a parameter by hand."""
        self._plan = None
        self._plan_params = None

    def _apply(self, fn, recurse=True):
        self.invalidate_plan()
        return super()._apply(fn, recurse)

    def _current_plan_key(self):
        """What the plan was built from, cheaply enough for every decode step: per parameter, which object holds it, where its
        storage is and its in-place version counter.  The (module, name) slots are listed once per plan (walking the module tree for
        them costs most of a millisecond at d26; looking the slots up again, some tens of microseconds), so a parameter object that
        is replaced -- `mod.weight = nn.Parameter(...)`, a swapped-in tensor -- changes the key like an in-place update does.  Only
        a replaced *module* needs invalidate_plan() (convert_to_float8_training, load_state_dict and .to() call it themselves)."""
        slots = self._plan_params
        if slots is None:
            slots = self._plan_params = [(mod, name, p) for mod in self.modules() for name, p in mod._parameters.items() if p is not None]
        key = []
        for mod, name, kept in slots:
            p = mod._parameters[name]
            if p is not kept:                    # (the kept reference also keeps the old object's id from being handed out again)
                self._plan_params = None
                return None                      # equal to no stored key: the plan is rebuilt and the slots are listed afresh
            key.append((p._version, p.data_ptr()))
        return tuple(key)

    def _build_plan(self):
        """Quantize every FP8 linear once, stack q|k|v, and fill the C descriptors."""
        cfg = self.config
        dev = self.get_device()
        if dev.type != "cuda":
            raise RuntimeError("GPT.forward runs on the GPU only: move the model to cuda (there is no CPU fallback)")
        for m in self._fp8_modules():
            if not isinstance(m, Float8Linear):
                raise RuntimeError("GPT.forward needs FP8 linears: call convert_to_float8_training(model, "
                                   "module_filter_fn=fp8_module_filter) first")
        D = cfg.n_embd // cfg.n_head
        if D != 128:
            raise ValueError(f"head_dim must be 128 on this path, got {D}")
        keep = []     # tensors the descriptors point into

        def q8(w):
            payload, inv, _ = ops.fp8_quantize(w.detach())
            return payload.view(torch.uint8), inv.reshape(1)

        def f32(t):
            t = t.detach().float().contiguous()
            keep.append(t)
            return t.data_ptr()

        def bf16(t):
            t = t.detach().to(torch.bfloat16).contiguous()
            keep.append(t)
            return t.data_ptr()

        layers = (_lib.LayerDesc * cfg.n_layer)()
        for i, blk in enumerate(self.transformer.h):
            parts = [q8(blk.attn.c_q.weight), q8(blk.attn.c_k.weight), q8(blk.attn.c_v.weight)]
            w_qkv = torch.cat([p[0] for p in parts], dim=0).contiguous()
            inv_qkv = torch.cat([p[1] for p in parts]).contiguous()
            w_ap, inv_ap = q8(blk.attn.c_proj.weight)
            w_fc, inv_fc = q8(blk.mlp.c_fc.weight)
            w_mp, inv_mp = q8(blk.mlp.c_proj.weight)
            keep += [w_qkv, inv_qkv, w_ap, inv_ap, w_fc, inv_fc, w_mp, inv_mp]
            ld = layers[i]
            ld.w_qkv, ld.inv_qkv = w_qkv.data_ptr(), inv_qkv.data_ptr()
            ld.w_attn_proj, ld.inv_attn_proj = w_ap.data_ptr(), inv_ap.data_ptr()
            ld.w_fc, ld.inv_fc = w_fc.data_ptr(), inv_fc.data_ptr()
            ld.w_mlp_proj, ld.inv_mlp_proj = w_mp.data_ptr(), inv_mp.data_ptr()
            if str(i) in self.value_embeds:
                ld.ve_table = bf16(self.value_embeds[str(i)].weight)
                ld.ve_gate_w = f32(blk.attn.ve_gate.weight)
            else:
                ld.ve_table, ld.ve_gate_w = None, None
            ld.window_left = int(self.window_sizes[i][0])
        w_lm, inv_lm = q8(self.lm_head.weight)
        cos, sin = self.rotary_tables(dev)
        keep += [w_lm, inv_lm, cos, sin]
        md = _lib.ModelDesc()
        md.n_layer, md.n_head, md.n_kv_head, md.n_embd = cfg.n_layer, cfg.n_head, cfg.n_kv_head, cfg.n_embd
        md.vocab_size, md.padded_vocab, md.rope_len = cfg.vocab_size, self.padded_vocab_size, self.rotary_seq_len
        md.softcap = self.SOFTCAP
        md.wte = bf16(self.transformer.wte.weight)
        md.w_lm_head, md.inv_lm_head = w_lm.data_ptr(), inv_lm.data_ptr()
        md.resid_lambdas, md.x0_lambdas = f32(self.resid_lambdas), f32(self.x0_lambdas)
        md.smear_w, md.smear_lambda = f32(self.smear_gate.weight.reshape(-1)), f32(self.smear_lambda)
        md.backout_lambda = f32(self.backout_lambda)
        md.cos, md.sin = cos.data_ptr(), sin.data_ptr()
        md.layers = C.cast(layers, C.POINTER(_lib.LayerDesc))
        self._plan = (md, layers, keep)
        self._workspaces = {}

    def _ensure_plan(self):
        key = self._current_plan_key()
        if self._plan is None or key is None or key != self._plan_key:
            self._build_plan()
            self._plan_key = self._current_plan_key()
        return self._plan[0]

    def _workspace(self, md, B, T, device):
        ws = self._workspaces.get((B, T))
        if ws is None:
            nbytes = _lib.lib().nc_gpt_workspace_bytes(C.byref(md), B, T)
            # prefill lengths vary: the table is bounded by the bytes it holds, not by its entry count
            held = sum(w.numel() for w in self._workspaces.values())
            if held + nbytes > self.WORKSPACE_CACHE_BYTES:
                self._workspaces.clear()
            ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=device)
            self._workspaces[(B, T)] = ws
        off = (-ws.data_ptr()) % 256
        return ws.data_ptr() + off, ws.numel() - off

    # -------------------------------------------------------------------------------------------
    @torch.no_grad()
    def _run(self, idx, kv_cache, last_only, taps=None):
        from .engine import KVCache
        cfg = self.config
        if not idx.is_cuda:
            raise RuntimeError("GPT.forward runs on the GPU only; there is no CPU fallback")
        B, T = idx.shape
        assert idx.dtype == torch.long
        if T > 1:
            # a prompt: worth one read-back to refuse ids outside the embedding table, as the reference's nn.Embedding does
            # (decode steps are fed by the sampler, or by the Engine's forced tokens, which it checks on the host; a direct
            # one-token call with a bad id is not caught and reads row 0 of the table)
            lo, hi = torch.aminmax(idx)
            if int(lo) < 0 or int(hi) >= self.padded_vocab_size:
                raise IndexError(f"token id out of range: [{int(lo)}, {int(hi)}] for an embedding table of {self.padded_vocab_size} rows")
        md = self._ensure_plan()
        if kv_cache is None:
            kv_cache = KVCache(B, cfg.n_kv_head, T, cfg.n_embd // cfg.n_head, cfg.n_layer, idx.device, torch.bfloat16)
        assert kv_cache.k_cache.dtype == torch.bfloat16, "the GPU path keeps the KV cache in bf16"
        assert kv_cache.batch_size == B and kv_cache.n_layers == cfg.n_layer and kv_cache.n_heads == cfg.n_kv_head
        pos_hi = getattr(kv_cache, "_pos_max", None)
        if pos_hi is None:
            pos_hi = int(kv_cache.cache_seqlens.max().item())
        assert pos_hi + T <= self.rotary_seq_len, f"Sequence length grew beyond the rotary embeddings cache: {pos_hi + T}"
        assert pos_hi + T <= kv_cache.max_seq_len, f"KV cache of {kv_cache.max_seq_len} tokens cannot take {pos_hi}+{T}"
        idx = idx.contiguous()
        rows = B if last_only else B * T
        logits = torch.empty(rows, cfg.vocab_size, dtype=torch.float32, device=idx.device)
        prev_in = kv_cache.prev_embedding
        if prev_in is not None:
            prev_in = prev_in.to(torch.bfloat16).contiguous()
        prev_out = torch.empty(B, 1, cfg.n_embd, dtype=torch.bfloat16, device=idx.device)
        cd = _lib.CacheDesc()
        cd.k_cache, cd.v_cache = kv_cache.k_cache.data_ptr(), kv_cache.v_cache.data_ptr()
        cd.cache_seqlens = kv_cache.cache_seqlens.data_ptr()
        cd.prev_in = prev_in.data_ptr() if prev_in is not None else None
        cd.prev_out = prev_out.data_ptr()
        cd.batch, cd.max_seq_len = B, kv_cache.max_seq_len
        # rows that begin with one replicated prompt and sit at one position (what Engine.generate builds): the cache may ask for the
        # shared start to be read once for all rows
        pos0 = getattr(kv_cache, "_pos0", None)
        shared = getattr(kv_cache, "shared_prefix_len", 0) if getattr(kv_cache, "share_prompt_reads", False) else 0
        uniform = T == 1 and pos0 is not None and pos0 == pos_hi and shared > 0 and pos0 >= shared
        cd.shared_prefix, cd.uniform_pos = (shared, pos0) if uniform else (0, 0)
        # a one-token step: the library advances the positions inside its last row kernel (one launch less per step)
        advance_inside = T == 1 and hasattr(kv_cache, "note_advanced") and cfg.n_embd % 8 == 0 and cfg.n_embd <= 8192
        cd.advance = T if advance_inside else 0
        ws_ptr, ws_bytes = self._workspace(md, B, T, idx.device)
        if taps is None:
            rc = _lib.lib().nc_gpt_forward(C.byref(md), C.byref(cd), idx.data_ptr(), B, T, logits.data_ptr(), 1 if last_only else 0,
                                           ws_ptr, ws_bytes, torch.cuda.current_stream().cuda_stream)
        else:
            taps["x"] = torch.empty(cfg.n_layer + 1, B, T, cfg.n_embd, dtype=torch.bfloat16, device=idx.device)
            taps["y"] = torch.empty(cfg.n_layer, B, T, cfg.n_head, cfg.n_embd // cfg.n_head, dtype=torch.bfloat16, device=idx.device)
            rc = _lib.lib().nc_gpt_forward_tapped(C.byref(md), C.byref(cd), idx.data_ptr(), B, T, logits.data_ptr(), 1 if last_only else 0,
                                                  ws_ptr, ws_bytes, taps["x"].data_ptr(), taps["y"].data_ptr(),
                                                  torch.cuda.current_stream().cuda_stream)
        _lib.check(rc)
        kv_cache.prev_embedding = prev_out
        if advance_inside:
            kv_cache.note_advanced(T)
        else:
            kv_cache.advance(T)
        return logits if last_only else logits.view(B, T, cfg.vocab_size)

    def forward(self, idx, targets=None, kv_cache=None, loss_reduction='mean'):
        """fp32 logits [B,T,vocab] (gpt.py:459-524).  The cache is appended in place and advanced by T."""
        if targets is not None:
            raise NotImplementedError("training loss is outside the inference path implemented here")
        return self._run(idx, kv_cache, last_only=False)

    def forward_last(self, idx, kv_cache=None):
        """Logits of the last position only, [B,vocab]: what Engine.generate consumes."""
        return self._run(idx, kv_cache, last_only=True)

    def forward_tapped(self, idx, kv_cache=None):
        """(logits [B,T,vocab], taps) for layer-by-layer comparisons: taps["x"] [L+1,B,T,E] holds the residual stream as each
        layer reads it (after the lambda mix, gpt.py:500) and, last, the final normalised rows (gpt.py:508); taps["y"]
        [L,B,T,H,D] the attention outputs before c_proj."""
        taps = {}
        return self._run(idx, kv_cache, last_only=False, taps=taps), taps

    # -------------------------------------------------------------------------------------------
    @torch.no_grad()
    def load_reference_state(self, state):
        """Load tensors keyed like the reference's state dict (e.g. an oracle parameter dict)."""
        own = self.state_dict()
        missing = [k for k in own if k not in state]
        extra = [k for k in state if k not in own]
        assert not missing and not extra, f"state mismatch: missing {missing[:3]} extra {extra[:3]}"
        for k, v in state.items():
            own[k].copy_(v.to(own[k].dtype))
        self.invalidate_plan()
