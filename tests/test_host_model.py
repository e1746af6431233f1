"""Host-side model logic that needs no GPU: GPT.init_weights against the reference's weights, and the cost accounting
(nanochat/gpt.py:341-388, scripts/infer_bench.py:51-53,130-138) against numbers the reference's own methods produced
(tests/golden/cost_accounting.json, written by tests/golden/make_golden.py) and against closed forms typed out here."""
import hashlib
import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from nanochat_amd import common                          # noqa: E402
from nanochat_amd.gpt import GPT, GPTConfig              # noqa: E402
from oracle import gpt_ref                               # noqa: E402

GOLD = os.path.join(os.path.dirname(__file__), "golden")
D4 = dict(sequence_len=2048, vocab_size=32768, n_layer=4, n_head=2, n_kv_head=2, n_embd=256)


def sha(t):
    t = t.detach().contiguous()
    raw = t.view(torch.int16).numpy().tobytes() if t.dtype == torch.bfloat16 else t.numpy().tobytes()
    return hashlib.sha256(raw).hexdigest()


def build_like_the_reference(cfg_kwargs, seed):
    """meta -> to_empty -> init_weights: how every reference caller builds the model
    (checkpoint_manager.py:99-104, scripts/base_train.py:141-151)."""
    with torch.device("meta"):
        model = GPT(GPTConfig(**cfg_kwargs))
    model.to_empty(device="cpu")
    torch.manual_seed(seed)
    model.init_weights()
    return model


def test_init_weights_reproduces_the_reference_weights():
    gold_name = "gpt_d4_bf16_fp8.json" if common.COMPUTE_DTYPE == torch.bfloat16 else "gpt_d4_fp32.json"
    if common.COMPUTE_DTYPE == torch.float16:
        pytest.skip("no golden for fp16")
    with open(os.path.join(GOLD, gold_name)) as f:
        gold = json.load(f)
    assert gold["config"] == D4
    model = build_like_the_reference(D4, seed=0)
    state = model.state_dict()
    want = gold["runs"]["repo"]["weight_sha256"]
    assert set(state) == set(want)
    # the oracle's restatement of the same recipe, tensor by tensor (tells a wrong distribution from a host whose RNG differs)
    params = gpt_ref.init_params(gpt_ref.GPTConfig(**D4), seed=0, compute_dtype=common.COMPUTE_DTYPE)
    for k, v in state.items():
        assert v.dtype == params[k].dtype and torch.equal(v, params[k]), k
    bad = [k for k in want if sha(state[k]) != want[k]]
    if len(bad) == len(want):
        pytest.skip("this host's torch RNG does not reproduce the golden weights")
    assert not bad, bad
    # structure the recipe promises (gpt.py:221-255)
    assert state["transformer.wte.weight"].dtype == common.COMPUTE_DTYPE
    assert state["value_embeds.1.weight"].dtype == common.COMPUTE_DTYPE
    assert state["lm_head.weight"].dtype == torch.float32
    for i in range(4):
        assert not state[f"transformer.h.{i}.attn.c_proj.weight"].any()
        assert not state[f"transformer.h.{i}.mlp.c_proj.weight"].any()
    assert state["smear_lambda"].item() == 0.0 and abs(state["backout_lambda"].item() - 0.2) < 1e-7
    assert torch.allclose(state["resid_lambdas"], torch.tensor([1.15, 1.15 - 0.1 / 3, 1.15 - 0.2 / 3, 1.05]))
    assert torch.allclose(state["x0_lambdas"], torch.tensor([0.20, 0.15, 0.10, 0.05]))


def test_init_weights_other_seed_and_shape_follow_the_oracle_recipe():
    kw = dict(sequence_len=256, vocab_size=1000, n_layer=5, n_head=4, n_kv_head=2, n_embd=512, window_pattern="SL")
    model = build_like_the_reference(kw, seed=7)
    params = gpt_ref.init_params(gpt_ref.GPTConfig(**kw), seed=7, compute_dtype=common.COMPUTE_DTYPE)
    state = model.state_dict()
    assert set(state) == set(params)
    for k, v in state.items():
        assert torch.equal(v, params[k]), k
    assert state["transformer.wte.weight"].shape[0] == 1024           # vocabulary padded to a multiple of 64 (gpt.py:170)


@pytest.fixture(scope="module")
def cost_gold():
    with open(os.path.join(GOLD, "cost_accounting.json")) as f:
        return json.load(f)


def meta_model(kw):
    with torch.device("meta"):
        return GPT(GPTConfig(**kw))


def test_cost_accounting_equals_the_reference_methods(cost_gold):
    from nanochat_amd.infer_bench import weight_bytes
    assert len(cost_gold["configs"]) >= 6
    for name, rec in cost_gold["configs"].items():
        model = meta_model(rec["config"])
        assert sum(p.numel() for p in model.parameters()) == rec["num_params"], name
        assert model.num_matmul_params() == rec["num_matmul_params"], name
        assert model.kv_bytes_per_token() == rec["kv_bytes_per_token"], name
        assert [list(w) for w in model.window_sizes] == rec["window_sizes"], name
        assert sorted(int(k) for k in model.value_embeds.keys()) == rec["value_embed_layers"], name
        for c, v in rec["kv_read_bytes"].items():
            assert model.kv_read_bytes(int(c)) == v, (name, c)
        for c, v in rec["estimate_decode_flops"].items():
            assert model.estimate_decode_flops(int(c)) == v, (name, c)
        for n, v in rec["estimate_prefill_flops"].items():
            assert model.estimate_prefill_flops(int(n)) == v, (name, n)
        # stored bytes with the embedding tables in bf16, everything else fp32: what the reference's weight_bytes()
        # gives on a freshly initialised model (scripts/infer_bench.py:51-53 on gpt.py:264-267)
        model.transformer.wte.to(torch.bfloat16)
        for ve in model.value_embeds.values():
            ve.to(torch.bfloat16)
        assert weight_bytes(model) == rec["weight_bytes_embeddings_in_compute_dtype"], name
        # the oracle's twins of the same quantities
        ocfg = gpt_ref.GPTConfig(**rec["config"])
        shapes = {k: torch.empty(v.shape, device="meta") for k, v in model.state_dict().items()}
        assert gpt_ref.num_matmul_params(shapes) == rec["num_matmul_params"], name
        assert gpt_ref.kv_bytes_per_token(ocfg) == rec["kv_bytes_per_token"], name
        for c, v in rec["estimate_decode_flops"].items():
            assert gpt_ref.estimate_decode_flops(ocfg, shapes, int(c)) == v, (name, c)
            assert gpt_ref.kv_read_bytes(ocfg, int(c)) == rec["kv_read_bytes"][c], (name, c)


def test_cost_accounting_counts_fp8_linears():
    """After the FP8 swap the reference's isinstance(m, Linear) count silently drops every converted layer
    (Float8Linear derives from nn.Linear, not gpt.Linear); here the count is unchanged by the swap."""
    from nanochat_amd.fp8 import Float8Linear, convert_to_float8_training, fp8_module_filter
    model = meta_model(D4)
    before = (model.num_matmul_params(), model.estimate_decode_flops(700), model.estimate_prefill_flops(700))
    convert_to_float8_training(model, module_filter_fn=fp8_module_filter)
    assert isinstance(model.lm_head, Float8Linear)
    assert (model.num_matmul_params(), model.estimate_decode_flops(700), model.estimate_prefill_flops(700)) == before


def test_cost_accounting_d26_closed_forms():
    """The headline shape by hand: E = 1664, 13 heads of 128, 26 layers, vocabulary 32768, windows SSSL."""
    E, L, H, D, V = 1664, 26, 13, 128, 32768
    model = meta_model(dict(sequence_len=2048, vocab_size=V, n_layer=L, n_head=H, n_kv_head=H, n_embd=E))
    n_ve = 13                                                      # layers 1, 3, ..., 25
    matmul = L * (4 * E * E + 8 * E * E) + V * E + n_ve * (H * 12) + 24
    assert model.num_matmul_params() == matmul == 918423556
    assert model.kv_bytes_per_token() == L * 2 * H * D * 2 == 173056
    long_layers = [i for i in range(L) if i % 4 == 3 or i == L - 1]
    assert long_layers == [3, 7, 11, 15, 19, 23, 25]
    per_key = 2 * H * D * 2                                        # K and V of one position, all heads, bf16
    assert model.kv_read_bytes(2048) == per_key * (7 * 2048 + 19 * 512) == 160169984
    assert model.kv_read_bytes(300) == per_key * 26 * 300
    assert 64 * model.kv_read_bytes(2048) == 10250878976           # the 10.25 GB a batch-64 step streams at full context
    attn = 4 * H * D * (7 * 1920 + 19 * 512)
    assert model.estimate_decode_flops(1920) == 2 * matmul + attn
    # prefill: a causal ramp up to the window, flat afterwards
    n = 1792
    ramp_long, ramp_short = n * (n + 1) // 2, 512 * 513 // 2 + (n - 512) * 512
    assert model.estimate_prefill_flops(n) == 2 * matmul * n + 4 * H * D * (7 * ramp_long + 19 * ramp_short)
    # infer_bench's ceiling at batch 1: every step re-reads the stored weights and the KV window (infer_bench.py:130-138)
    from nanochat_amd.infer_bench import static_card
    card = static_card(model, prompt_len=1792, decode_tokens=256, total_vram=288 * 2**30, peak_bw=8.0e12)
    assert card["context_mid"] == 1920
    assert card["kv_read_bytes_per_step"] == per_key * (7 * 1920 + 19 * 512)
    assert card["ceiling_bs1_tok_per_sec"] == round(8.0e12 / (card["weight_bytes"] + card["kv_read_bytes_per_step"]), 1)
    assert card["max_full_context_rows"] == int((288 * 2**30 - card["weight_bytes"]) / (173056 * 2048))
    assert card["param_dtypes"] == {"float32": card["num_params"]}
