"""KV cache, next-token sampler and the batched generation loop, API-compatible with nanochat/engine.py
(KVCache :82-137, sample_next_token :140-156, Engine :169-299, calculator :25-79).

Device work (model forward, sampling on GPU logits) goes to the HIP kernels; this file is host logic:
cache bookkeeping, the per-row tool-use state machine and the streaming generator protocol.
"""
import signal
import warnings
from collections import deque
from contextlib import contextmanager

import torch
import torch.nn.functional as F

from . import ops
from .common import COMPUTE_DTYPE

# ------------------------------------------------------------------------------------------------
# Calculator tool (engine.py:25-79): evaluates the text between <|python_start|> and <|python_end|>.
_MATH_CHARS = set("0123456789*+-/.() ")
_TEXT_CHARS = set("abcdefghijklmnopqrstuvwxyzABCDEFGHIJKLMNOPQRSTUVWXYZ0123456789'\"()._ ")
_BANNED = ("__", "import", "exec", "eval", "compile", "open", "file", "input", "raw_input", "globals", "locals",
           "vars", "dir", "getattr", "setattr", "delattr", "hasattr")


class _CalcTimeout(Exception):
    pass


@contextmanager
def _alarm(seconds, what):
    def on_alarm(signum, frame):
        raise _CalcTimeout(f"'{what}': timed out after {seconds} seconds")
    signal.signal(signal.SIGALRM, on_alarm)
    signal.alarm(seconds)
    try:
        yield
    finally:
        signal.alarm(0)


def eval_with_timeout(formula, max_time=3):
    """eval() with empty builtins under a SIGALRM limit; None on any failure."""
    try:
        with _alarm(max_time, formula), warnings.catch_warnings():
            warnings.simplefilter("ignore", SyntaxWarning)
            return eval(formula, {"__builtins__": {}}, {})
    except Exception:
        return None


def use_calculator(expr):
    """Arithmetic over + - * / ( ) (no **), or a quoted-string .count(...) expression; else None."""
    expr = expr.replace(",", "")
    if set(expr) <= _MATH_CHARS:
        return None if "**" in expr else eval_with_timeout(expr)
    if not set(expr) <= _TEXT_CHARS:
        return None
    lowered = expr.lower()
    if any(word in lowered for word in _BANNED):
        return None
    if ".count(" not in expr:
        return None
    return eval_with_timeout(expr)


# ------------------------------------------------------------------------------------------------
class KVCache:
    """Pre-allocated (n_layers, B, T, H, D) key and value tensors in FA3 layout, per-row lengths in an
    int32 tensor, and the previous token's normalised embedding for the smear gate (engine.py:82-137).

    A host-side copy of the position is kept so that get_pos() does not have to read the device tensor
    back every decode step; it is exact as long as positions change only through advance/reset/prefill
    (or set_seqlens for ragged batches, where it tracks row 0 like the reference's get_pos)."""

    def __init__(self, batch_size, num_heads, seq_len, head_dim, num_layers, device, dtype, prefill_from=None, share_prompt_reads=False):
        """prefill_from (not in the reference's signature): another cache whose tokens this one starts with, i.e.
        KVCache(...) followed by .prefill(prefill_from) in one step.  On the GPU the tensors then never get the zero fill that the
        copy would overwrite anyway (at d26 / 64 rows / 1792 prompt tokens that fill is 20 of the 22.7 GB, 4 ms of the time to the
        first token): only the positions past the prompt are cleared, and the end state is the same.

        share_prompt_reads (not in the reference's signature, off by default): after a prefill from a batch-1 cache every row holds a
        copy of the same prompt.  With this set the cache remembers how long that shared start is (`shared_prefix_len`) and a one-token
        forward reads it once for all rows in the layers that see most of it, instead of once per row; the tensors keep the reference's
        layout and contents.  The promise that goes with it: nobody writes into positions [0, shared_prefix_len) of k_cache / v_cache
        by hand (set shared_prefix_len = 0 first)."""
        self.batch_size = batch_size
        self.max_seq_len = seq_len
        self.n_layers = num_layers
        self.n_heads = num_heads
        self.head_dim = head_dim
        shape = (num_layers, batch_size, seq_len, num_heads, head_dim)
        lazy = prefill_from is not None and torch.device(device).type == "cuda"
        alloc = torch.empty if lazy else torch.zeros
        self.k_cache = alloc(shape, device=device, dtype=dtype)
        self.v_cache = alloc(shape, device=device, dtype=dtype)
        self.cache_seqlens = torch.zeros(batch_size, dtype=torch.int32, device=device)
        self.prev_embedding = None
        self._pos0 = 0          # host mirror of cache_seqlens[0]
        self._pos_max = 0       # host mirror of cache_seqlens.max()
        self.share_prompt_reads = bool(share_prompt_reads)
        self.shared_prefix_len = 0      # positions [0, this) hold the same bytes in every row (set by prefill from a batch-1 cache)
        if prefill_from is not None:
            if lazy:
                n = prefill_from.get_pos()
                assert seq_len >= prefill_from.max_seq_len >= n
                self.k_cache[:, :, n:].zero_()
                self.v_cache[:, :, n:].zero_()
            self.prefill(prefill_from)

    def reset(self):
        self.cache_seqlens.zero_()
        self.prev_embedding = None
        self._pos0 = self._pos_max = 0
        self.shared_prefix_len = 0

    def get_pos(self):
        return self._pos0

    def get_layer_cache(self, layer_idx):
        return self.k_cache[layer_idx], self.v_cache[layer_idx]

    def advance(self, num_tokens):
        self.cache_seqlens += num_tokens
        self._pos0 += num_tokens
        self._pos_max += num_tokens

    def note_advanced(self, num_tokens):
        """The forward call advanced `cache_seqlens` on the device itself (nc_cache_desc.advance): only the host mirrors follow."""
        self._pos0 += num_tokens
        self._pos_max += num_tokens

    def rewind(self, num_tokens, prev_embedding):
        """Take back the last advance (the appended rows stay in the tensors and are overwritten by the next
        append at the same positions); `prev_embedding` is the smear state from before that forward."""
        assert 0 < num_tokens <= self._pos0
        self.cache_seqlens -= num_tokens
        self._pos0 -= num_tokens
        self._pos_max -= num_tokens
        self.prev_embedding = prev_embedding
        if self._pos0 < self.shared_prefix_len:         # the next append would land inside the shared start
            self.shared_prefix_len = 0

    def set_seqlens(self, seqlens):
        """Ragged rows: install per-row lengths (host list or tensor)."""
        t = torch.as_tensor(seqlens, dtype=torch.int32)
        assert t.shape == (self.batch_size,)
        self._pos0, self._pos_max = int(t[0]), int(t.max())
        assert 0 <= int(t.min()) and self._pos_max <= self.max_seq_len
        self.cache_seqlens.copy_(t)
        self.shared_prefix_len = 0

    def prefill(self, other):
        """Copy another cache's first pos tokens into every row of this one (engine.py:123-137)."""
        assert self.get_pos() == 0, "Cannot prefill a non-empty KV cache"
        assert self.n_layers == other.n_layers and self.n_heads == other.n_heads and self.head_dim == other.head_dim
        assert self.max_seq_len >= other.max_seq_len
        n = other.get_pos()
        if self.k_cache.is_cuda:
            assert other.batch_size in (1, self.batch_size)
            ops.kv_cache_prefill(self.k_cache, other.k_cache, n)
            ops.kv_cache_prefill(self.v_cache, other.v_cache, n)
        else:           # host-side caches (the engine's own logic under test with a mock model)
            self.k_cache[:, :, :n, :, :] = other.k_cache[:, :, :n, :, :]
            self.v_cache[:, :, :n, :, :] = other.v_cache[:, :, :n, :, :]
        self.cache_seqlens.fill_(n)
        self._pos0 = self._pos_max = n
        self.shared_prefix_len = n if (other.batch_size == 1 and self.batch_size > 1) else 0
        if other.prev_embedding is not None:
            self.prev_embedding = other.prev_embedding.expand(self.batch_size, -1, -1).clone()


# ------------------------------------------------------------------------------------------------
@torch.inference_mode()
def sample_next_token(logits, rng, temperature=1.0, top_k=None):
    """(B, vocab) logits -> (B, 1) token ids (engine.py:140-156).

    GPU logits: the HIP sampler; the Exp(1) variates of the multinomial draw come from `rng`.
    CPU logits (host-side tests with a mock model): the same steps in torch."""
    assert temperature >= 0.0, "temperature must be non-negative"
    if logits.is_cuda:
        logits = logits.float()
        if temperature == 0.0:
            return ops.sample(logits, 0.0, None, None)
        B, V = logits.shape
        k = min(top_k, V) if (top_k is not None and top_k > 0) else V
        noise = torch.empty(B, k, dtype=torch.float32, device=logits.device).exponential_(1.0, generator=rng)
        return ops.sample(logits, temperature, top_k, noise)
    if temperature == 0.0:
        return torch.argmax(logits, dim=-1, keepdim=True)
    if top_k is not None and top_k > 0:
        vals, idx = torch.topk(logits, min(top_k, logits.size(-1)), dim=-1)
        choice = torch.multinomial(F.softmax(vals / temperature, dim=-1), num_samples=1, generator=rng)
        return idx.gather(1, choice)
    return torch.multinomial(F.softmax(logits / temperature, dim=-1), num_samples=1, generator=rng)


# ------------------------------------------------------------------------------------------------
class RowState:
    """Generation state of one batch row (engine.py:160-167)."""

    def __init__(self, current_tokens=None):
        self.current_tokens = current_tokens or []
        self.forced_tokens = deque()
        self.in_python_block = False
        self.python_expr_tokens = []
        self.completed = False


class _Specials:
    def __init__(self, tokenizer):
        self.python_start = tokenizer.encode_special("<|python_start|>")
        self.python_end = tokenizer.encode_special("<|python_end|>")
        self.output_start = tokenizer.encode_special("<|output_start|>")
        self.output_end = tokenizer.encode_special("<|output_end|>")
        self.assistant_end = tokenizer.encode_special("<|assistant_end|>")
        self.bos = tokenizer.get_bos_token_id()


class Engine:
    def __init__(self, model, tokenizer):
        self.model = model
        self.tokenizer = tokenizer

    def _step_row(self, state, sampled, sp):
        """Pick the row's next token (forced beats sampled), update the tool-use machine.
        Returns (token, mask) with mask 0 for forced and 1 for sampled (engine.py:238-267)."""
        forced = len(state.forced_tokens) > 0
        token = state.forced_tokens.popleft() if forced else sampled
        state.current_tokens.append(token)
        if token == sp.assistant_end or token == sp.bos:
            state.completed = True
        if token == sp.python_start:
            state.in_python_block = True
            state.python_expr_tokens = []
        elif token == sp.python_end and state.in_python_block:
            state.in_python_block = False
            if state.python_expr_tokens:
                result = use_calculator(self.tokenizer.decode(state.python_expr_tokens))
                if result is not None:
                    state.forced_tokens.append(sp.output_start)
                    state.forced_tokens.extend(self.tokenizer.encode(str(result)))
                    state.forced_tokens.append(sp.output_end)
            state.python_expr_tokens = []
        elif state.in_python_block:
            state.python_expr_tokens.append(token)
        return token, (0 if forced else 1)

    def _last_logits(self, ids, kv_cache):
        fast = getattr(self.model, "forward_last", None)
        if fast is not None:
            return fast(ids, kv_cache=kv_cache)
        return self.model.forward(ids, kv_cache=kv_cache)[:, -1, :]

    @torch.inference_mode()
    def generate(self, tokens, num_samples=1, max_tokens=None, temperature=1.0, top_k=None, seed=42, share_prompt_reads=False):
        """One batch-1 prefill, cache replicated to num_samples rows, then streamed decoding.
        Yields (token_column, token_masks) per step (engine.py:175-275).

        share_prompt_reads (not in the reference's signature, off by default): every row's cache starts with a copy of the same
        prompt; with this set, the decode steps read that prompt once for all rows in the full-context layers (see KVCache)."""
        assert isinstance(tokens, list) and isinstance(tokens[0], int), "expecting list of ints"
        device = self.model.get_device()
        dtype = torch.bfloat16 if torch.device(device).type == "cuda" else COMPUTE_DTYPE
        rng = torch.Generator(device=device)
        rng.manual_seed(seed)
        sp = _Specials(self.tokenizer)

        cfg = self.model.config
        geometry = dict(num_heads=cfg.n_kv_head, head_dim=cfg.n_embd // cfg.n_head, num_layers=cfg.n_layer)
        kv_prefill = KVCache(batch_size=1, seq_len=len(tokens), device=device, dtype=dtype, **geometry)
        ids = torch.tensor([tokens], dtype=torch.long, device=device)
        logits = self._last_logits(ids, kv_prefill).expand(num_samples, -1)

        hint = (len(tokens) + max_tokens) if max_tokens is not None else cfg.sequence_len
        kv_decode = KVCache(batch_size=num_samples, seq_len=hint, device=device, dtype=dtype, prefill_from=kv_prefill,
                            share_prompt_reads=share_prompt_reads, **geometry)
        del kv_prefill

        rows = [RowState(tokens.copy()) for _ in range(num_samples)]
        produced = 0
        # On the GPU the next forward is enqueued on the sampled ids before the host has seen them: the ids travel to a
        # pinned buffer by an async copy placed ahead of that forward, and the tool-use state machine runs while the
        # GPU computes.  If the machine then forces a different token for some row, the step is taken back (positions
        # and smear state) and redone with the forced column -- the outputs are those of the plain loop.
        ahead = torch.device(device).type == "cuda" and hasattr(self.model, "forward_last")
        if ahead:
            host_ids = torch.empty(num_samples, dtype=torch.long, pin_memory=True)
            ids_ready = torch.cuda.Event()
        while True:
            if max_tokens is not None and produced >= max_tokens:
                break
            if all(r.completed for r in rows):
                break
            sampled_dev = sample_next_token(logits, rng, temperature, top_k)
            # (not in front of the first token: the caller gets it as soon as it is sampled, as in the reference's loop, where the
            # time to the first token ends before the first decode forward)
            run_ahead = ahead and produced > 0 and not (max_tokens is not None and produced + 1 >= max_tokens)
            if run_ahead:
                # (on the launch stream: handing this copy to a stream of its own costs 90 us per step -- with a second queue
                # active every one of the step's ~190 launches starts ~0.5 us later)
                host_ids.copy_(sampled_dev[:, 0], non_blocking=True)
                ids_ready.record()
                prev_before = kv_decode.prev_embedding
                logits_ahead = self._last_logits(sampled_dev, kv_decode)
                ids_ready.synchronize()
                sampled = host_ids.tolist()
            else:
                sampled = sampled_dev[:, 0].tolist()
            column, masks = [], []
            for r, s in zip(rows, sampled):
                tok, mask = self._step_row(r, s, sp)
                column.append(tok)
                masks.append(mask)
            yield column, masks
            produced += 1
            if run_ahead and column == sampled:
                logits = logits_ahead
                continue
            if run_ahead:
                kv_decode.rewind(1, prev_before)
            # forced tokens come from the tokenizer, not from the sampler: refuse what the embedding table does not hold
            rows_in_table = getattr(self.model, "padded_vocab_size", None)
            if rows_in_table is not None and not all(0 <= t < rows_in_table for t in column):
                raise IndexError(f"token id out of range for an embedding table of {rows_in_table} rows: {column}")
            ids = torch.tensor(column, dtype=torch.long, device=device).unsqueeze(1)
            logits = self._last_logits(ids, kv_decode)

    def generate_batch(self, tokens, num_samples=1, **kwargs):
        """Drain generate(); returns (sequences, masks) without terminal tokens (engine.py:277-299)."""
        sp = _Specials(self.tokenizer)
        results = [tokens.copy() for _ in range(num_samples)]
        masks = [[0] * len(tokens) for _ in range(num_samples)]
        done = [False] * num_samples
        for column, column_masks in self.generate(tokens, num_samples, **kwargs):
            for i, (tok, mask) in enumerate(zip(column, column_masks)):
                if done[i]:
                    continue
                if tok == sp.assistant_end or tok == sp.bos:
                    done[i] = True
                else:
                    results[i].append(tok)
                    masks[i].append(mask)
            if all(done):
                break
        return results, masks
