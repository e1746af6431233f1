"""Synthetic stand-ins for what needs the network or a trained checkpoint: a model of a given depth with random
weights, and a tokenizer with the four methods the Engine uses.  Throughput does not depend on the weights."""
import torch

from .fp8 import convert_to_float8_training, fp8_module_filter
from .gpt import GPT, GPTConfig


def config_for_depth(depth, sequence_len=2048, vocab_size=32768, window_pattern="SSSL", aspect_ratio=64, head_dim=128,
                     n_kv_head=None):
    """The reference's depth -> shape rule (scripts/base_train.py:129-141): dim = depth * 64 rounded up to head_dim."""
    model_dim = -(-(depth * aspect_ratio) // head_dim) * head_dim
    n_head = model_dim // head_dim
    return GPTConfig(sequence_len=sequence_len, vocab_size=vocab_size, n_layer=depth, n_head=n_head,
                     n_kv_head=n_kv_head or n_head, n_embd=model_dim, window_pattern=window_pattern)


def random_init_model(cfg, device, seed=0):
    """Random weights drawn on the device with the distributions of the reference's init_weights (gpt.py:204-268), but
    with non-zero output projections, gates and lambdas so that every kernel does real work.  bf16, FP8 linears."""
    with torch.device("meta"):
        model = GPT(cfg)
    model.to_empty(device=device)
    g = torch.Generator(device=device).manual_seed(seed)
    s = 3 ** 0.5 * cfg.n_embd ** -0.5
    with torch.no_grad():
        for name, p in model.named_parameters():
            if name.endswith("wte.weight"):
                p.normal_(0.0, 0.8, generator=g)
            elif name == "lm_head.weight":
                p.normal_(0.0, 0.03, generator=g)
            elif "value_embeds" in name or "c_q" in name or "c_k" in name or "c_v" in name or "attn.c_proj" in name:
                p.uniform_(-s, s, generator=g)
            elif "c_fc" in name:
                p.uniform_(-0.4 * s, 0.4 * s, generator=g)
            elif "mlp.c_proj" in name:
                p.uniform_(-0.5 * s, 0.5 * s, generator=g)
            elif "gate" in name:
                p.uniform_(-0.5, 0.5, generator=g)
            elif name == "resid_lambdas":
                p.copy_(torch.linspace(1.15, 1.05, cfg.n_layer))
            elif name == "x0_lambdas":
                p.copy_(torch.linspace(0.20, 0.05, cfg.n_layer))
            elif name == "smear_lambda":
                p.fill_(0.35)
            elif name == "backout_lambda":
                p.fill_(0.2)
            else:
                raise RuntimeError(f"unhandled parameter {name}")
        model.to(torch.bfloat16)
    model.eval()
    convert_to_float8_training(model, module_filter_fn=fp8_module_filter)
    return model


class SyntheticTokenizer:
    """encode_special / get_bos_token_id / encode / decode: the Engine's whole view of a tokenizer (engine.py:186-192).
    The specials sit outside the vocabulary, so sampling from a random model never ends a row early."""

    def encode_special(self, s):
        return 1 << 30

    def get_bos_token_id(self):
        return (1 << 30) + 1

    def encode(self, s, prepend=None):
        return []

    def decode(self, tokens):
        return ""
