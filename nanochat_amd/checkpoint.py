"""Build the GPU model from a nanochat checkpoint directory (nanochat/checkpoint_manager.py:41-114).

Layout written by the reference's save_checkpoint: `model_%06d.pt` (the state dict: `transformer.wte.weight`,
`transformer.h.{i}.attn.c_q.weight`, ..., `resid_lambdas`, `x0_lambdas`, `smear_gate.weight`, `smear_lambda`,
`backout_lambda`, `value_embeds.{i}.weight`, `lm_head.weight`) and `meta_%06d.json` with a `model_config` dict.
Only tensors are read from the .pt file (`weights_only=True`: nothing in it is executed).  The tokenizer and
the optimizer shards are not part of this path.
"""
import glob
import json
import os
import re

import torch

from .fp8 import convert_to_float8_training, fp8_module_filter
from .gpt import GPT, GPTConfig


def find_last_step(checkpoint_dir):
    """Largest step with a model file (checkpoint_manager.py:139-146)."""
    steps = [int(m.group(1)) for f in glob.glob(os.path.join(checkpoint_dir, "model_*.pt"))
             if (m := re.search(r"model_(\d+)\.pt$", f))]
    if not steps:
        raise FileNotFoundError(f"No checkpoints found in {checkpoint_dir}")
    return max(steps)


def load_checkpoint(checkpoint_dir, step, device):
    """(state dict, meta dict) of one step."""
    model_path = os.path.join(checkpoint_dir, f"model_{step:06d}.pt")
    meta_path = os.path.join(checkpoint_dir, f"meta_{step:06d}.json")
    model_data = torch.load(model_path, map_location=device, weights_only=True)
    with open(meta_path, "r", encoding="utf-8") as f:
        meta_data = json.load(f)
    return model_data, meta_data


def build_model(checkpoint_dir, step=None, device="cuda"):
    """GPT on `device` holding the checkpoint's tensors as saved, FP8 linears swapped in with the reference's filter
    (scripts/base_train.py:178-185).  Returns (model, meta).

    The reference evaluates a checkpoint with plain Linear modules (bf16 matmuls, checkpoint_manager.py:99-104); the path built
    here is the quantized one only, so a loaded model always runs its block linears and lm_head as e4m3 Float8Linear -- the
    numerics of the reference's --fp8 training forward, not of its bf16 evaluation."""
    if step is None:
        step = find_last_step(checkpoint_dir)
    device = torch.device(device)
    model_data, meta = load_checkpoint(checkpoint_dir, step, device)
    # a compiled model saves its keys with this prefix (checkpoint_manager.py:93)
    model_data = {k.removeprefix("_orig_mod."): v for k, v in model_data.items()}
    cfg_kwargs = dict(meta["model_config"])
    cfg_kwargs.setdefault("window_pattern", "L")          # checkpoints from before sliding windows
    config = GPTConfig(**cfg_kwargs)
    if "resid_lambdas" not in model_data:                  # older checkpoints: identity residual scaling, no x0 mix
        model_data["resid_lambdas"] = torch.ones(config.n_layer)
    if "x0_lambdas" not in model_data:
        model_data["x0_lambdas"] = torch.zeros(config.n_layer)
    with torch.device("meta"):
        model = GPT(config)
    own = model.state_dict()
    missing = sorted(set(own) - set(model_data))
    unexpected = sorted(set(model_data) - set(own))
    if missing or unexpected:
        raise RuntimeError(f"checkpoint does not match the model: missing {missing[:4]}, unexpected {unexpected[:4]}")
    for k, v in model_data.items():
        if own[k].shape != v.shape:
            raise RuntimeError(f"{k}: checkpoint shape {tuple(v.shape)} != model shape {tuple(own[k].shape)}")
    # The checkpoint's tensors become the parameters, in the dtypes they were saved in (load_state_dict(strict=True,
    # assign=True) at checkpoint_manager.py:104): fp32 master weights are quantized to e4m3 from fp32, as the reference's
    # Float8Linear would do on every call.
    model.load_state_dict({k: v.to(device) for k, v in model_data.items()}, strict=True, assign=True)
    model.eval()
    convert_to_float8_training(model, module_filter_fn=fp8_module_filter)
    return model, meta
