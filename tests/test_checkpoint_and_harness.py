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
        # the tensors are taken over as saved (load_state_dict(assign=True), checkpoint_manager.py:104)
        assert got[k].dtype == want[k].dtype and torch.equal(got[k], want[k]), k
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
    model, _ = build_model(d, 5, device="cpu")
    assert model.config.window_pattern == "L"                      # checkpoint_manager.py:22-27
    assert torch.equal(model.resid_lambdas.float(), torch.ones(3)) and torch.equal(model.x0_lambdas.float(), torch.zeros(3))
    bad = str(tmp_path / "bad")
    write_checkpoint(bad, 1, drop=("smear_lambda",))
    with pytest.raises(RuntimeError, match="missing"):
        build_model(bad, 1, device="cpu")
    with pytest.raises(FileNotFoundError):
        find_last_step(str(tmp_path))


def write_reference_style_checkpoint(d, step, cfg, seed):
    """A checkpoint as the reference's training writes one: the state dict of a model with fp32 master weights and
    bf16 embedding tables (gpt.py:264-267), here with every sub-layer active."""
    from oracle import gpt_ref
    params = gpt_ref.init_params(gpt_ref.GPTConfig(**cfg), seed=seed, compute_dtype=torch.bfloat16, trained_like=True)
    os.makedirs(d, exist_ok=True)
    torch.save({"_orig_mod." + k: v for k, v in params.items()}, os.path.join(d, f"model_{step:06d}.pt"))
    with open(os.path.join(d, f"meta_{step:06d}.json"), "w") as f:
        json.dump({"step": step, "model_config": cfg}, f)


@pytest.mark.gpu
def test_checkpoint_model_matches_the_oracle_on_the_same_file(tmp_path):
    """The same model_*.pt goes into the HIP model through build_model and, tensor for tensor, into the CPU oracle:
    prefill and decode logits must agree as closely as two reference-equivalent oracle variants agree with each other."""
    from nanochat_amd.engine import KVCache
    from oracle import decode_ref, gpt_ref
    from test_gpu_gpt import assert_within_floor, oracle_floor
    cfg = dict(sequence_len=256, vocab_size=1024, n_layer=3, n_head=2, n_kv_head=1, n_embd=256, window_pattern="SL")
    d = str(tmp_path / "ck")
    write_reference_style_checkpoint(d, 7, cfg, seed=21)
    model, meta = build_model(d, device="cuda")
    assert meta["step"] == 7
    assert model.lm_head.weight.dtype == torch.float32 and model.transformer.wte.weight.dtype == torch.bfloat16
    state = torch.load(os.path.join(d, "model_000007.pt"), map_location="cpu", weights_only=True)
    state = {k.removeprefix("_orig_mod."): v for k, v in state.items()}
    rt = gpt_ref.Runtime(gpt_ref.GPTConfig(**cfg), state, compute_dtype=torch.bfloat16, fp8=True)
    g = torch.Generator().manual_seed(1)
    prompt = torch.randint(0, 1024, (2, 19), generator=g)
    steps = [torch.randint(0, 1024, (2, 1), generator=g) for _ in range(4)]

    def run(r):
        c = decode_ref.new_cache(r.cfg, 2, 32, torch.bfloat16)
        outs = [gpt_ref.forward(r, prompt, c)]
        for nxt in steps:
            outs.append(gpt_ref.forward(r, nxt, c))
        return torch.cat(outs, dim=1)
    floor_rel, floor_max, want, want_def = oracle_floor(rt, run)
    kv = KVCache(2, 1, 32, 128, 3, "cuda", torch.bfloat16)
    got = [model(prompt.cuda(), kv_cache=kv).cpu()]
    for nxt in steps:
        got.append(model(nxt.cuda(), kv_cache=kv).cpu())
    got = torch.cat(got, dim=1)
    assert_within_floor(got, want, want_def, floor_rel, floor_max, "checkpoint -> HIP model vs checkpoint -> oracle")
    # the weights the GPU streams are the e4m3 bytes the oracle's quantizer makes of the file's fp32 tensors
    from nanochat_amd import ops
    from oracle import fp8_ref
    for key, mod in (("lm_head.weight", model.lm_head), ("transformer.h.1.mlp.c_proj.weight", model.transformer.h[1].mlp.c_proj)):
        w8, inv, _ = fp8_ref.to_fp8(state[key])
        payload, inv_gpu, _ = ops.fp8_quantize(mod.weight.detach())
        assert torch.equal(payload.cpu().view(torch.uint8), w8.view(torch.uint8)), key
        assert inv_gpu.cpu().view(torch.int32).item() == inv.reshape(()).view(torch.int32).item(), key


@pytest.mark.gpu
def test_infer_bench_card_and_json_line():
    from nanochat_amd import infer_bench
    from nanochat_amd.synthetic import config_for_depth
    buf = io.StringIO()
    with contextlib.redirect_stdout(buf):
        infer_bench.main(["--depth", "2", "--prompt-tokens", "40", "--decode-tokens", "6", "--batch-sizes", "1,3"])
    lines = buf.getvalue().strip().splitlines()
    card = json.loads(lines[-1])
    for key in ("source", "step", "model_config", "gpu", "peak_bandwidth_bytes_per_sec", "total_vram_bytes", "num_params", "param_dtypes",
                "weight_bytes", "kv_bytes_per_token", "kv_read_bytes_per_step", "context_mid", "peak_flops_per_sec",
                "decode_flops_per_token", "ceiling_bs1_tok_per_sec", "max_full_context_rows", "prompt_tokens", "decode_tokens",
                "temperature", "prefill", "sweep"):                      # every key of the reference's card (infer_bench.py:158-180)
        assert key in card, key
    # the static card against the reference's formulas (infer_bench.py:130-138) worked out by hand for this shape:
    # depth 2 -> dim 128, one head, vocabulary 32768, windows (512, 2048); bf16 parameters
    cfg = config_for_depth(2)
    assert (cfg.n_embd, cfg.n_head, cfg.n_layer) == (128, 1, 2) and card["model_config"]["n_embd"] == 128
    E, V = 128, 32768
    n_matmul = 2 * 12 * E * E + V * E + 12 + 24                 # blocks, lm_head, one value-embedding gate, smear gate
    n_params = n_matmul + V * E + V * E + 2 + 2 + 1 + 1         # + wte, one value embedding, lambdas
    assert card["num_params"] == n_params and card["param_dtypes"] == {"bfloat16": n_params}
    assert card["weight_bytes"] == 2 * n_params
    assert card["kv_bytes_per_token"] == 2 * 2 * 1 * 128 * 2
    assert card["context_mid"] == 40 + 3 and card["prompt_tokens"] == 40 and card["decode_tokens"] == 6
    assert card["kv_read_bytes_per_step"] == 2 * (2 * 128 * 2) * 43
    assert card["decode_flops_per_token"] == 2 * n_matmul + 2 * 4 * 1 * 128 * 43
    assert card["peak_bandwidth_bytes_per_sec"] == 8.0e12 and card["peak_flops_per_sec"] == 2.5e15
    assert card["ceiling_bs1_tok_per_sec"] == round(8.0e12 / (card["weight_bytes"] + card["kv_read_bytes_per_step"]), 1)
    assert card["max_full_context_rows"] == int((card["total_vram_bytes"] - card["weight_bytes"]) / (card["kv_bytes_per_token"] * 2048))
    assert [s["batch_size"] for s in card["sweep"]] == [1, 3]
    for s in card["sweep"]:
        assert s["decode_steps"] == 5 and s["tok_per_sec"] > 0 and s["tpot_sec"] > 0 and 0 < s["mbu_percent"] < 100
        # MBU / MFU by the reference's definitions (infer_bench.py:215-222) from the card's own numbers
        mbu = 100 * ((card["weight_bytes"] + s["batch_size"] * card["kv_read_bytes_per_step"]) / s["tpot_sec"]) / 8.0e12
        mfu = 100 * (s["batch_size"] * card["decode_flops_per_token"] / s["tpot_sec"]) / 2.5e15
        assert abs(s["mbu_percent"] - mbu) <= 0.02 * mbu + 0.01 and abs(s["mfu_percent"] - mfu) <= 0.02 * mfu + 1e-4
    assert card["prefill"]["tok_per_sec"] > 0
