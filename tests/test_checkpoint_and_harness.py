"""The checkpoint loader (nanochat/checkpoint_manager.py:41-114 restated) and the infer_bench harness."""
import contextlib
import io
import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

from nanochat_amd.checkpoint import build_model, find_last_step, load_checkpoint   # noqa: E402
from nanochat_amd.gpt import GPT, GPTConfig                                         # noqa: E402

CFG = dict(sequence_len=256, vocab_size=1024, n_layer=3, n_head=2, n_kv_head=1, n_embd=256, window_pattern="SL")


def write_checkpoint(tmp_path, step, drop=(), prefix="", cfg=CFG):
    torch.manual_seed(step)
    model = GPT(GPTConfig(**cfg))
    with torch.no_grad():
        for p in model.parameters():
            p.normal_(0.0, 0.05)
    state = {prefix + k: v.clone() for k, v in model.state_dict().items() if k not in drop}
    os.makedirs(tmp_path, exist_ok=True)
    torch.save(state, os.path.join(tmp_path, f"model_{step:06d}.pt"))
    meta_cfg = {k: v for k, v in cfg.items()}
    with open(os.path.join(tmp_path, f"meta_{step:06d}.json"), "w") as f:
        json.dump({"step": step, "model_config": meta_cfg}, f)
    return model


def test_loader_reads_the_reference_layout(tmp_path):
    d = str(tmp_path / "d3")
    write_checkpoint(d, 10)
    src = write_checkpoint(d, 250, prefix="_orig_mod.")           # a compiled model's keys
    assert find_last_step(d) == 250
    state, meta = load_checkpoint(d, 250, "cpu")
    assert meta["step"] == 250 and all(k.startswith("_orig_mod.") for k in state)
    model, meta = build_model(d, device="cpu")
    assert meta["model_config"] == CFG and model.config == GPTConfig(**CFG)
    want = src.state_dict()
    got = model.state_dict()
    assert set(got) == set(want)
    for k in want:
        assert got[k].dtype == torch.bfloat16
        assert torch.equal(got[k], want[k].bfloat16()), k
    # the reference's filter converts every block linear and lm_head, not the gates (scripts/base_train.py:178-185)
    from nanochat_amd.fp8 import Float8Linear
    assert isinstance(model.lm_head, Float8Linear) and isinstance(model.transformer.h[0].mlp.c_fc, Float8Linear)
    assert not isinstance(model.smear_gate, Float8Linear)


def test_loader_patches_old_checkpoints_and_rejects_mismatches(tmp_path):
    d = str(tmp_path / "old")
    old_cfg = {k: v for k, v in CFG.items() if k != "window_pattern"}
    write_checkpoint(d, 5, drop=("resid_lambdas", "x0_lambdas"))
    with open(os.path.join(d, "meta_000005.json"), "w") as f:
        json.dump({"step": 5, "model_config": old_cfg}, f)
    model, _ = build_model(d, 5, device="cpu", fp8=False)
    assert model.config.window_pattern == "L"                      # checkpoint_manager.py:22-27
    assert torch.equal(model.resid_lambdas.float(), torch.ones(3)) and torch.equal(model.x0_lambdas.float(), torch.zeros(3))
    bad = str(tmp_path / "bad")
    write_checkpoint(bad, 1, drop=("smear_lambda",))
    with pytest.raises(RuntimeError, match="missing"):
        build_model(bad, 1, device="cpu")
    with pytest.raises(FileNotFoundError):
        find_last_step(str(tmp_path))


@pytest.mark.gpu
def test_checkpoint_model_matches_the_model_it_was_saved_from(tmp_path):
    from nanochat_amd.engine import KVCache
    from nanochat_amd.fp8 import convert_to_float8_training, fp8_module_filter
    d = str(tmp_path / "ck")
    src = write_checkpoint(d, 7)
    src = src.to("cuda").to(torch.bfloat16)
    convert_to_float8_training(src, module_filter_fn=fp8_module_filter)
    loaded, _ = build_model(d, 7, device="cuda")
    ids = torch.randint(0, 1024, (2, 19), generator=torch.Generator().manual_seed(1)).cuda()
    outs = []
    for m in (src, loaded):
        kv = KVCache(2, 1, 32, 128, 3, "cuda", torch.bfloat16)
        outs.append(m.forward(ids, kv_cache=kv))
    assert torch.equal(outs[0], outs[1])


@pytest.mark.gpu
def test_infer_bench_card_and_json_line():
    from nanochat_amd import infer_bench
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        infer_bench.main(["--depth", "2", "--prompt-tokens", "40", "--decode-tokens", "6", "--batch-sizes", "1,3"])
    lines = buf.getvalue().strip().splitlines()
    card = json.loads(lines[-1])
    for key in ("model_config", "gpu", "peak_bandwidth_bytes_per_sec", "weight_bytes", "kv_bytes_per_token", "kv_read_bytes_per_step",
                "context_mid", "decode_flops_per_token", "ceiling_bs1_tok_per_sec", "prompt_tokens", "decode_tokens", "prefill", "sweep"):
        assert key in card, key
    assert [s["batch_size"] for s in card["sweep"]] == [1, 3]
    for s in card["sweep"]:
        assert s["decode_steps"] == 5 and s["tok_per_sec"] > 0 and s["tpot_sec"] > 0 and 0 < s["mbu_percent"] < 100
    assert card["prefill"]["tok_per_sec"] > 0
