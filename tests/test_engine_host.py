"""Host logic of the product Engine / KVCache, restating the reference's tests/test_engine.py
(:84-267) against nanochat_amd.engine with the same mock model and byte tokenizer, plus the
tool-use state machine and calculator (engine.py:46-79, 238-267).  CPU only."""
from dataclasses import dataclass

import pytest
import torch

from nanochat_amd.engine import Engine, KVCache, use_calculator


@dataclass
class MockConfig:
    n_kv_head: int = 4
    n_head: int = 4
    n_embd: int = 64
    n_layer: int = 2
    sequence_len: int = 128


class MockModel:
    """Uniform logits; advances the cache like a real forward does."""

    def __init__(self, vocab_size=262, script=None):
        self.vocab_size = vocab_size
        self.config = MockConfig()
        self._device = torch.device("cpu")
        self.script = list(script) if script else None   # optional forced argmax sequence
        self.calls = 0

    def get_device(self):
        return self._device

    def forward(self, ids, kv_cache=None):
        B, T = ids.shape
        if kv_cache is not None:
            kv_cache.advance(T)
        logits = torch.zeros(B, T, self.vocab_size)
        if self.script is not None:
            tok = self.script[min(self.calls, len(self.script) - 1)]
            logits[:, -1, tok] = 10.0
            self.calls += 1
        return logits


class ByteTokenizer:
    def __init__(self):
        self._special = {"<|python_start|>": 256, "<|python_end|>": 257, "<|output_start|>": 258,
                         "<|output_end|>": 259, "<|assistant_end|>": 260, "<|bos|>": 261}

    def encode_special(self, s):
        return self._special[s]

    def get_bos_token_id(self):
        return 261

    def encode(self, s, prepend=None):
        toks = list(s.encode("utf-8"))
        return ([prepend] + toks) if prepend is not None else toks

    def decode(self, tokens):
        return bytes(t for t in tokens if t < 256).decode("utf-8", errors="replace")


PROMPT = [261, 72, 101, 108, 108, 111]


def test_kv_cache_basic():
    kv = KVCache(batch_size=2, num_heads=3, seq_len=64, head_dim=5, num_layers=6, device="cpu", dtype=torch.float32)
    assert kv.get_pos() == 0
    assert kv.k_cache.shape == (6, 2, 64, 3, 5) and kv.v_cache.shape == (6, 2, 64, 3, 5)
    kv.advance(10)
    assert kv.get_pos() == 10
    kv.advance(5)
    assert kv.get_pos() == 15 and kv.cache_seqlens.tolist() == [15, 15]
    kv.reset()
    assert kv.get_pos() == 0 and kv.cache_seqlens.tolist() == [0, 0]
    k0, v0 = kv.get_layer_cache(0)
    assert k0.shape == (2, 64, 3, 5) and v0.shape == (2, 64, 3, 5)
    assert k0.data_ptr() == kv.k_cache.data_ptr()          # a view, so in-place appends land in the cache


def test_kv_cache_prefill():
    src = KVCache(batch_size=1, num_heads=4, seq_len=32, head_dim=8, num_layers=2, device="cpu", dtype=torch.float32)
    src.k_cache[0, 0, :16] = 1.0
    src.v_cache[0, 0, :16] = 2.0
    src.prev_embedding = torch.full((1, 1, 32), 3.0)
    src.advance(16)
    dst = KVCache(batch_size=3, num_heads=4, seq_len=64, head_dim=8, num_layers=2, device="cpu", dtype=torch.float32)
    dst.prefill(src)
    assert dst.get_pos() == 16 and dst.cache_seqlens.tolist() == [16, 16, 16]
    assert (dst.k_cache[0, :, :16] == 1.0).all() and (dst.v_cache[0, :, :16] == 2.0).all()
    assert (dst.k_cache[0, :, 16:] == 0).all()
    assert dst.prev_embedding.shape == (3, 1, 32) and (dst.prev_embedding == 3.0).all()
    with pytest.raises(AssertionError):
        dst.prefill(src)                                    # non-empty destination
    small = KVCache(batch_size=1, num_heads=4, seq_len=8, head_dim=8, num_layers=2, device="cpu", dtype=torch.float32)
    with pytest.raises(AssertionError):
        small.prefill(src)                                  # destination shorter than the source


def test_multi_sample_first_token_diversity():
    engine = Engine(MockModel(vocab_size=262), ByteTokenizer())
    first = None
    for column, masks in engine.generate(PROMPT, num_samples=16, max_tokens=1, temperature=1.0, seed=42):
        first = column
    assert len(first) == 16 and len(set(first)) > 1


def test_seed_reproducibility():
    engine = Engine(MockModel(), ByteTokenizer())
    for seed in [1, 42, 123, 999]:
        r1, _ = engine.generate_batch(PROMPT, max_tokens=5, seed=seed)
        r2, _ = engine.generate_batch(PROMPT, max_tokens=5, seed=seed)
        r3, _ = engine.generate_batch(PROMPT, max_tokens=5, seed=seed)
        assert r1 == r2 == r3


def test_temperature_zero_determinism():
    engine = Engine(MockModel(), ByteTokenizer())
    r1, _ = engine.generate_batch(PROMPT, temperature=0.0, max_tokens=5, seed=1)
    r2, _ = engine.generate_batch(PROMPT, temperature=0.0, max_tokens=5, seed=42)
    r3, _ = engine.generate_batch(PROMPT, temperature=0.0, max_tokens=5, seed=123)
    assert r1 == r2 == r3


def test_max_tokens_respected():
    engine = Engine(MockModel(), ByteTokenizer())
    for max_tokens in [1, 4, 16, 64]:
        results, _ = engine.generate_batch(PROMPT, max_tokens=max_tokens)
        assert len(results[0]) - len(PROMPT) <= max_tokens


def test_num_samples_count():
    engine = Engine(MockModel(), ByteTokenizer())
    for n in [1, 4, 16, 64]:
        results, masks = engine.generate_batch(PROMPT, num_samples=n, max_tokens=3)
        assert len(results) == n and len(masks) == n


def test_different_seeds_introduce_variation_when_temperature_nonzero():
    engine = Engine(MockModel(), ByteTokenizer())
    outs = set()
    for seed in [1, 42, 123, 999, 1000, 1001, 1002, 1003, 1004, 1005]:
        results, _ = engine.generate_batch(PROMPT, temperature=1.0, max_tokens=5, seed=seed)
        outs.add(tuple(results[0]))
    assert len(outs) > 1


def test_calculator_closed_forms():
    assert use_calculator("1+2*3") == 7
    assert use_calculator("1,000 + 24") == 1024
    assert use_calculator("2**10") is None                 # power operator refused
    assert use_calculator("'strawberry'.count('r')") == 3
    assert use_calculator("__import__('os')") is None
    assert use_calculator("'a'.upper()") is None           # only .count( is allowed
    assert use_calculator("1/0") is None                   # exceptions give None
    assert use_calculator("abc") is None


def test_tool_use_forces_calculator_output():
    # greedy script: <|python_start|> '2' '+' '3' <|python_end|> then anything; the engine must force
    # <|output_start|> '5' <|output_end|> with mask 0 and stop on <|assistant_end|>
    script = [256, ord("2"), ord("+"), ord("3"), 257, 65, 65, 65, 260]
    engine = Engine(MockModel(script=script), ByteTokenizer())
    cols, masks = [], []
    for column, m in engine.generate(PROMPT, num_samples=1, max_tokens=12, temperature=0.0):
        cols.append(column[0])
        masks.append(m[0])
    assert cols[:5] == [256, 50, 43, 51, 257]
    assert cols[5:8] == [258, ord("5"), 259] and masks[5:8] == [0, 0, 0]
    assert all(m == 1 for m in masks[:5])
    assert cols[-1] == 260                                  # generation stops after the terminal token
    results, rmasks = Engine(MockModel(script=script), ByteTokenizer()).generate_batch(PROMPT, max_tokens=12, temperature=0.0)
    assert 260 not in results[0] and len(results[0]) == len(rmasks[0])


def test_gpu_only_modules_refuse_cpu_tensors():
    from nanochat_amd import ops
    from nanochat_amd.fp8 import Float8Linear, Float8LinearConfig, convert_to_float8_training, fp8_module_filter
    with pytest.raises(RuntimeError):
        ops.fp8_quantize(torch.zeros(16, dtype=torch.bfloat16))
    lin = torch.nn.Linear(128, 256, bias=False)
    seq = torch.nn.Sequential(lin, torch.nn.Linear(12, 2, bias=False))
    convert_to_float8_training(seq, module_filter_fn=fp8_module_filter)
    assert isinstance(seq[0], Float8Linear) and not isinstance(seq[1], Float8Linear)
    assert seq[0].weight is lin.weight
    with pytest.raises(RuntimeError):
        seq[0](torch.zeros(2, 128))
    with pytest.raises(ValueError):
        Float8LinearConfig.from_recipe_name("rowwise")
    assert isinstance(Float8LinearConfig.from_recipe_name("tensorwise"), Float8LinearConfig)
