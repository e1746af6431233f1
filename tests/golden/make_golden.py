"""Writes the golden fixtures in this directory by running the reference itself.

Run in the authoring container only (the reference tree is not shipped anywhere):

    python tests/golden/make_golden.py quantize
    python tests/golden/make_golden.py gpt_fp32
    NANOCHAT_DTYPE=bfloat16 python tests/golden/make_golden.py gpt_bf16_fp8
    NANOCHAT_DTYPE=bfloat16 python tests/golden/make_golden.py cost

What is imported from the reference: ``nanochat.fp8`` (``_to_fp8``, ``Float8Linear``,
``convert_to_float8_training``), ``nanochat.gpt`` (``GPT``, ``GPTConfig``) and,
through it, ``nanochat.flash_attention``.  ``nanochat.engine`` is not imported (its
import chain needs packages that are absent here); the KV-cache container handed
to the reference's ``GPT.forward`` is this repo's oracle container, which has the
same attributes.  Only the two things nothing else pins are taken from these
runs: exact end-to-end logits / greedy ids of the composed model, and the
quantizer's output on awkward inputs.  Fixtures are inputs and expected outputs
(ids, logit samples, payload bytes, hashes), never weights or source.
"""
import hashlib
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, "/root/reference")


def sha(t):
    t = t.detach().contiguous()
    if t.dtype == torch.bfloat16:
        raw = t.view(torch.int16).numpy().tobytes()
    else:
        raw = t.numpy().tobytes()
    return hashlib.sha256(raw).hexdigest()


# ----------------------------------------------------------------------------------------
def quantize_cases():
    """Named awkward inputs, each fully determined by its recipe."""
    g = torch.Generator().manual_seed(1234)
    cases = {}
    cases["zeros_bf16"] = torch.zeros(64, dtype=torch.bfloat16)
    cases["single_one_bf16"] = torch.tensor([0.0, 1.0, 0.0, -0.0], dtype=torch.bfloat16)
    x = torch.randn(4096, generator=g)
    x[::997] *= 20.0
    cases["normal_outliers_bf16"] = x.bfloat16()
    cases["normal_fp32"] = torch.randn(1024, generator=g)
    # amax = 448 makes scale exactly 1: payload is the plain e4m3 rounding of the input
    ties = torch.tensor([448.0, -448.0, 17.0, 19.0, 21.0, 23.0, 1.0625, 1.1875, 0.001953125,
                         0.0009765625, 0.0029296875, 0.00146484375, 447.0, 431.9, 432.0, 464.0 / 2,
                         -17.0, -0.001953125, 0.0, 3.0e-5], dtype=torch.float32)
    cases["scale_one_ties_fp32"] = ties
    cases["scale_one_ties_bf16"] = ties.bfloat16()
    cases["tiny_amax_fp32"] = torch.tensor([1e-20, -3e-21, 0.0], dtype=torch.float32)
    cases["below_floor_fp32"] = torch.tensor([1e-13, -5e-14], dtype=torch.float32)
    cases["huge_fp32"] = torch.tensor([3.0e38, -1.0e38, 1.0, 1e30], dtype=torch.float32)
    u = (torch.rand(2048, generator=g) * 2 - 1) * (3 / 1664) ** 0.5
    cases["uniform_weight_bf16"] = u.bfloat16()
    return cases


def tensor_bits(t):
    if t.dtype == torch.bfloat16:
        return {"dtype": "bf16", "bits": t.view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()}
    return {"dtype": "f32", "bits": t.view(torch.int32).to(torch.int64).bitwise_and(0xFFFFFFFF).tolist()}


def make_quantize():
    from nanochat.fp8 import _to_fp8
    out = {}
    for name, x in quantize_cases().items():
        payload, inv = _to_fp8(x, torch.float8_e4m3fn)
        out[name] = {
            "input": tensor_bits(x),
            "payload": payload.view(torch.uint8).tolist(),
            "inv_scale_bits": int(inv.view(torch.int32).item()) & 0xFFFFFFFF,
        }
    with open(os.path.join(HERE, "quantize_reference.json"), "w") as f:
        json.dump(out, f)
    print("wrote quantize_reference.json", {k: len(v["payload"]) for k, v in out.items()})


# ----------------------------------------------------------------------------------------
def build_reference_model(cfg_kwargs, seed, state=None):
    from nanochat.gpt import GPT, GPTConfig
    cfg = GPTConfig(**cfg_kwargs)
    with torch.device("meta"):
        model = GPT(cfg)
    model.to_empty(device="cpu")
    torch.manual_seed(seed)
    model.init_weights()
    if state is not None:
        missing = model.load_state_dict(state, strict=True)
    model.eval()
    return model


def logits_digest(logits_row):
    """A compact, order-sensitive sample of one fp32 logits row."""
    top = torch.topk(logits_row, 8)
    return {
        "head": logits_row[:32].tolist(),
        "strided": logits_row[::1021].tolist(),
        "top_idx": top.indices.tolist(),
        "top_val": top.values.tolist(),
    }


def run_reference_decode(model, prompt, max_tokens, compute_dtype):
    """Prefill at B=1 then greedy decode with the reference's GPT.forward(kv_cache=...)."""
    from oracle.decode_ref import RefKVCache
    cfg = model.config
    cache = RefKVCache(1, cfg.n_kv_head, len(prompt) + max_tokens, cfg.n_embd // cfg.n_head,
                       cfg.n_layer, compute_dtype)
    ids = torch.tensor([prompt], dtype=torch.long)
    steps = []
    tokens = []
    with torch.inference_mode():
        logits = model.forward(ids, kv_cache=cache)[:, -1, :]
        for _ in range(max_tokens):
            row = logits[0].float()
            nxt = int(torch.argmax(row).item())
            top2 = torch.topk(row, 2).values
            steps.append({"digest": logits_digest(row), "margin": float(top2[0] - top2[1])})
            tokens.append(nxt)
            logits = model.forward(torch.tensor([[nxt]], dtype=torch.long), kv_cache=cache)[:, -1, :]
    return tokens, steps


def make_gpt(tag, fp8):
    from nanochat.common import COMPUTE_DTYPE
    from oracle import gpt_ref
    cfg_kwargs = dict(sequence_len=2048, vocab_size=32768, n_layer=4, n_head=2, n_kv_head=2, n_embd=256)
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, 32768, (32,), generator=g).tolist()
    out = {"config": cfg_kwargs, "prompt": prompt, "compute_dtype": str(COMPUTE_DTYPE), "fp8": fp8, "runs": {}}
    for init in ("repo", "trained_like"):
        seed = 0
        if init == "repo":
            model = build_reference_model(cfg_kwargs, seed)
        else:
            params = gpt_ref.init_params(gpt_ref.GPTConfig(**cfg_kwargs), seed=seed,
                                         compute_dtype=COMPUTE_DTYPE, trained_like=True)
            model = build_reference_model(cfg_kwargs, seed, state=params)
        hashes = {k: sha(v) for k, v in model.state_dict().items()}
        if fp8:
            import torch.nn as nn
            from nanochat.fp8 import convert_to_float8_training

            def filt(mod, fqn):
                return (isinstance(mod, nn.Linear) and mod.in_features % 16 == 0 and mod.out_features % 16 == 0
                        and min(mod.in_features, mod.out_features) >= 128)
            convert_to_float8_training(model, module_filter_fn=filt)
        n_tok = 64
        tokens, steps = run_reference_decode(model, prompt, n_tok, COMPUTE_DTYPE)
        run = {"weight_sha256": hashes, "greedy_ids": tokens, "steps": steps}
        if not fp8 and init == "repo":
            # the cache-free greedy decode of the reference (gpt.py:526-555)
            run["nocache_ids"] = list(model.generate(prompt, max_tokens=16, temperature=0.0))
        out["runs"][init] = run
        print(tag, init, "ids", tokens[:16], "min margin", min(s["margin"] for s in steps))
    with open(os.path.join(HERE, f"{tag}.json"), "w") as f:
        json.dump(out, f)
    print("wrote", tag)


# ----------------------------------------------------------------------------------------
COST_CONFIGS = {
    "d4": dict(sequence_len=2048, vocab_size=32768, n_layer=4, n_head=2, n_kv_head=2, n_embd=256),
    "d20": dict(sequence_len=2048, vocab_size=32768, n_layer=20, n_head=10, n_kv_head=10, n_embd=1280),
    "d26": dict(sequence_len=2048, vocab_size=32768, n_layer=26, n_head=13, n_kv_head=13, n_embd=1664),
    "d26_L": dict(sequence_len=2048, vocab_size=32768, n_layer=26, n_head=13, n_kv_head=13, n_embd=1664, window_pattern="L"),
    "d32_gqa": dict(sequence_len=2048, vocab_size=32768, n_layer=32, n_head=16, n_kv_head=4, n_embd=2048),
    "odd_vocab": dict(sequence_len=1024, vocab_size=50257, n_layer=5, n_head=3, n_kv_head=1, n_embd=384, window_pattern="SL"),
}
COST_CONTEXTS = (1, 512, 513, 1920, 2048)
COST_PROMPTS = (1, 400, 512, 1792, 2048)


def make_cost():
    """The reference's own cost accounting (gpt.py:341-388, scripts/infer_bench.py:51-53,130-138) on models that
    exist on the meta device only (no weights are materialised), before any FP8 conversion."""
    from nanochat.common import COMPUTE_DTYPE
    from nanochat.gpt import GPT, GPTConfig
    assert COMPUTE_DTYPE == torch.bfloat16
    out = {"compute_dtype": str(COMPUTE_DTYPE), "configs": {}}
    for name, kw in COST_CONFIGS.items():
        with torch.device("meta"):
            model = GPT(GPTConfig(**kw))
        # the dtypes a loaded checkpoint has in the reference: everything as built (fp32), embeddings in the compute dtype
        # (gpt.py:264-267); element sizes follow from that without materialising a weight
        emb = {id(model.transformer.wte.weight)} | {id(ve.weight) for ve in model.value_embeds.values()}
        w_bytes = sum(p.numel() * (COMPUTE_DTYPE.itemsize if id(p) in emb else p.element_size()) for p in model.parameters())
        rec = {
            "config": kw,
            "num_params": sum(p.numel() for p in model.parameters()),
            "num_matmul_params": model.num_matmul_params(),
            "weight_bytes_embeddings_in_compute_dtype": w_bytes,
            "kv_bytes_per_token": model.kv_bytes_per_token(),
            "window_sizes": [list(w) for w in model.window_sizes],
            "value_embed_layers": sorted(int(k) for k in model.value_embeds.keys()),
            "kv_read_bytes": {str(c): model.kv_read_bytes(c) for c in COST_CONTEXTS},
            "estimate_decode_flops": {str(c): model.estimate_decode_flops(c) for c in COST_CONTEXTS},
            "estimate_prefill_flops": {str(n): model.estimate_prefill_flops(n) for n in COST_PROMPTS},
        }
        out["configs"][name] = rec
        print(name, rec["num_params"], rec["num_matmul_params"], rec["kv_bytes_per_token"])
    with open(os.path.join(HERE, "cost_accounting.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote cost_accounting.json")


if __name__ == "__main__":
    mode = sys.argv[1]
    if mode == "quantize":
        make_quantize()
    elif mode == "gpt_fp32":
        assert os.environ.get("NANOCHAT_DTYPE") is None
        make_gpt("gpt_d4_fp32", fp8=False)
    elif mode == "gpt_bf16_fp8":
        assert os.environ.get("NANOCHAT_DTYPE") == "bfloat16"
        make_gpt("gpt_d4_bf16_fp8", fp8=True)
    elif mode == "cost":
        assert os.environ.get("NANOCHAT_DTYPE") == "bfloat16"
        make_cost()
    else:
        raise SystemExit(f"unknown mode {mode}")
