"""Inference benchmark card and batch-size sweep, the counterpart of the reference's scripts/infer_bench.py:
time to first token, median time per output token, tokens/s, MBU and MFU per decode batch size, a static card of
what the architecture costs, and -- as the very last line of stdout -- one JSON document with the same data
(same field names as the reference's card, so scripts written against it keep working).

    python -m nanochat_amd.infer_bench --depth 26                      # random weights of the d26 shape
    python -m nanochat_amd.infer_bench --checkpoint-dir DIR [--step N] # a nanochat checkpoint

Accounting follows the reference (scripts/infer_bench.py:51-53,130-138,215-222): a decode step moves the stored
weights plus batch * kv_read_bytes(context_mid); MBU is that over the median step time over the peak bandwidth;
MFU uses estimate_decode_flops / estimate_prefill_flops over the peak of common.get_peak_flops (the bf16 figure, as
in the reference's table).  Every reference field keeps the reference's definition.  Added beside them, under
names of their own: what a step really streams here (the cached e4m3 copies of the FP8 linears, one byte per
element: `weight_bytes_streamed`, `ceiling_bs1_streamed_tok_per_sec`, `mbu_streamed_percent`) and MFU against the
fp8 dense peak (`mfu_fp8_percent`).  Random prompts are used when there is no tokenizer.
"""
import argparse
import json
import time

import torch

from .common import PEAK_FP8_FLOPS, get_peak_bandwidth, get_peak_flops
from .engine import Engine
from .synthetic import SyntheticTokenizer, config_for_depth, random_init_model


def weight_bytes(model):
    """Bytes of parameters as stored (scripts/infer_bench.py:51-53)."""
    return sum(p.numel() * p.element_size() for p in model.parameters())


def streamed_weight_bytes(model):
    """What a decode step reads: e4m3 payloads of the FP8 linears, bf16 for the remaining small matrices.  Embedding
    tables are gathered (a few rows per step) and not counted."""
    from .fp8 import Float8Linear
    fp8 = {id(m.weight) for m in model._fp8_modules() if isinstance(m, Float8Linear)}
    total = 0
    for name, p in model.named_parameters():
        if "wte" in name or "value_embeds" in name:
            continue
        total += p.numel() * (1 if id(p) in fp8 else p.element_size())
    return total


def static_card(model, prompt_len, decode_tokens, total_vram, peak_bw):
    """What the architecture costs before anything is measured (scripts/infer_bench.py:124-138,160-176), as the
    fields of the JSON card: parameter counts per dtype, stored weight bytes, KV bytes stored per token and read per
    step at the representative context prompt + decode/2, the batch-1 ceiling peak_bw / (weights + KV read), and how
    many full-context rows fit next to the weights."""
    config = model.config
    w_bytes = weight_bytes(model)
    dtype_counts = {}
    for p in model.parameters():
        name = str(p.dtype).replace("torch.", "")
        dtype_counts[name] = dtype_counts.get(name, 0) + p.numel()
    kv_store = model.kv_bytes_per_token()
    context_mid = prompt_len + decode_tokens // 2
    kv_read = model.kv_read_bytes(context_mid)
    w_stream = streamed_weight_bytes(model)
    return {
        "num_params": sum(p.numel() for p in model.parameters()), "param_dtypes": dtype_counts, "weight_bytes": w_bytes,
        "weight_bytes_streamed": w_stream, "kv_bytes_per_token": kv_store, "kv_read_bytes_per_step": kv_read,
        "context_mid": context_mid, "decode_flops_per_token": model.estimate_decode_flops(context_mid),
        "ceiling_bs1_tok_per_sec": round(peak_bw / (w_bytes + kv_read), 1),
        "ceiling_bs1_streamed_tok_per_sec": round(peak_bw / (w_stream + kv_read), 1),
        "max_full_context_rows": int((total_vram - w_bytes) / (kv_store * config.sequence_len)),
    }


def bench_generate(engine, prompt_tokens, batch_size, decode_tokens, temperature, share_prompt_reads=False):
    """One timed generation with the reference's protocol: the first next() is the time to first token (batch-1
    prefill, cache replication, first sample, first forward), every further next() is one decode step, each
    followed by a device synchronisation."""
    device = engine.model.get_device()
    torch.cuda.reset_peak_memory_stats(device)
    torch.cuda.synchronize(device)
    gen = engine.generate(prompt_tokens, num_samples=batch_size, max_tokens=decode_tokens, temperature=temperature,
                          share_prompt_reads=share_prompt_reads)
    t0 = time.perf_counter()
    next(gen)
    torch.cuda.synchronize(device)
    ttft = time.perf_counter() - t0
    step_times = []
    while True:
        t1 = time.perf_counter()
        try:
            next(gen)
        except StopIteration:
            break
        torch.cuda.synchronize(device)
        step_times.append(time.perf_counter() - t1)
    return dict(ttft=ttft, step_times=step_times, peak_vram=torch.cuda.max_memory_allocated(device))


def main(argv=None):
    ap = argparse.ArgumentParser(description="Inference benchmark (MI355X, FP8 linears, KV-cache decode)")
    ap.add_argument("--checkpoint-dir", type=str, default=None, help="nanochat checkpoint directory (model_*.pt, meta_*.json)")
    ap.add_argument("-s", "--step", type=int, default=None, help="checkpoint step (default: last)")
    ap.add_argument("--depth", type=int, default=26, help="without a checkpoint: random weights of this depth")
    ap.add_argument("--window-pattern", type=str, default="SSSL")
    ap.add_argument("--n-kv-head", type=int, default=None)
    ap.add_argument("--prompt-tokens", type=int, default=2048)
    ap.add_argument("--decode-tokens", type=int, default=256)
    ap.add_argument("--batch-sizes", type=str, default="1,8,32,128")
    ap.add_argument("-t", "--temperature", type=float, default=0.0)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--share-prompt-reads", action="store_true",
                    help="not in the reference: read the prompt that Engine.generate replicates into every row once for all rows")
    args = ap.parse_args(argv)
    assert torch.cuda.is_available(), "infer_bench needs the GPU"
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.checkpoint_dir:
        from .checkpoint import build_model
        model, meta = build_model(args.checkpoint_dir, args.step, device)
        source, step, model_config = "checkpoint", meta.get("step"), meta["model_config"]
    else:
        cfg = config_for_depth(args.depth, window_pattern=args.window_pattern, n_kv_head=args.n_kv_head)
        model = random_init_model(cfg, device, args.seed)
        source, step, model_config = f"random-init d{args.depth}", None, dict(vars(cfg))
    config = model.config
    engine = Engine(model, SyntheticTokenizer())

    prompt_len = min(args.prompt_tokens, config.sequence_len - args.decode_tokens)
    if prompt_len < args.prompt_tokens:
        print(f"note: clamping prompt to {prompt_len} tokens so prompt+decode fits sequence_len={config.sequence_len}")
    g = torch.Generator().manual_seed(args.seed)
    prompt = torch.randint(0, config.vocab_size, (prompt_len,), generator=g).tolist()

    device_name = torch.cuda.get_device_name(device)
    peak_bw, peak_flops = get_peak_bandwidth(device_name), get_peak_flops(device_name)
    total_vram = torch.cuda.get_device_properties(device).total_memory
    card = static_card(model, prompt_len, args.decode_tokens, total_vram, peak_bw)
    w_bytes, w_stream, kv_read, context_mid = card["weight_bytes"], card["weight_bytes_streamed"], card["kv_read_bytes_per_step"], card["context_mid"]

    bar = "=" * 100
    print(bar)
    print(f"Model: {source} | depth {config.n_layer}, dim {config.n_embd}, heads {config.n_head}, kv heads {config.n_kv_head}")
    print(f"GPU: {device_name} | peak bandwidth {peak_bw / 1e12:.2f} TB/s | peak compute {peak_flops / 1e12:.0f} TFLOPS "
          f"(fp8 dense {PEAK_FP8_FLOPS / 1e12:.0f}) | VRAM {total_vram / 2**30:.0f} GiB")
    param_dtypes = ", ".join(f"{n:,} {name}" for name, n in sorted(card["param_dtypes"].items()))
    print(f"Parameters: {card['num_params']:,} ({param_dtypes}) | weight bytes as stored: {w_bytes / 2**20:.0f} MiB | streamed per "
          f"decode step {w_stream / 2**20:.0f} MiB (e4m3 linears)")
    print(f"KV cache: {card['kv_bytes_per_token']:,} bytes/token stored | {kv_read:,} bytes read/step at context {context_mid} "
          f"(window pattern {config.window_pattern})")
    print(f"Theoretical decode ceiling at batch 1: {card['ceiling_bs1_tok_per_sec']:,.0f} tok/s ({card['ceiling_bs1_streamed_tok_per_sec']:,.0f} "
          f"on the bytes really streamed) | max ~{card['max_full_context_rows']:,} full-context rows in VRAM")
    print(bar)
    payload = {
        "source": source, "step": step, "model_config": model_config, "gpu": device_name,
        "peak_bandwidth_bytes_per_sec": peak_bw, "total_vram_bytes": total_vram, **card,
        "peak_flops_per_sec": peak_flops, "peak_fp8_flops_per_sec": PEAK_FP8_FLOPS,
        "prompt_tokens": prompt_len, "decode_tokens": args.decode_tokens, "temperature": args.temperature,
        "share_prompt_reads": bool(args.share_prompt_reads), "sweep": [],
    }

    bench_generate(engine, prompt, 1, 2, args.temperature)                  # warm-up (weight plan, workspaces)
    pre = bench_generate(engine, prompt, 1, 2, args.temperature)
    prefill_mfu = 100 * model.estimate_prefill_flops(prompt_len) / pre["ttft"] / peak_flops
    print(f"Prefill (batch 1, {prompt_len} tokens): {prompt_len / pre['ttft']:,.0f} tok/s | MFU {prefill_mfu:.1f}%")
    payload["prefill"] = {"tok_per_sec": round(prompt_len / pre["ttft"], 1), "mfu_percent": round(prefill_mfu, 2),
                          "mfu_fp8_percent": round(prefill_mfu * peak_flops / PEAK_FP8_FLOPS, 2), "time_sec": round(pre["ttft"], 6)}

    header = f"{'batch':>6} {'TTFT ms':>9} {'TPOT ms':>9} {'tok/s':>10} {'MBU %':>7} {'MFU %':>7} {'VRAM GiB':>9} {'steps':>6}"
    print(header)
    print("-" * len(header))
    for batch_size in [int(b) for b in args.batch_sizes.split(",")]:
        bench_generate(engine, prompt, batch_size, 8, args.temperature, args.share_prompt_reads)     # warm-up at this batch size
        res = bench_generate(engine, prompt, batch_size, args.decode_tokens, args.temperature, args.share_prompt_reads)
        steps = res["step_times"]
        if not steps:
            print(f"{batch_size:>6}  no decode steps")
            continue
        tpot = sorted(steps)[len(steps) // 2]
        tok_per_sec = batch_size * len(steps) / sum(steps)
        mbu = 100 * ((w_bytes + batch_size * kv_read) / tpot) / peak_bw
        mbu_streamed = 100 * ((w_stream + batch_size * kv_read) / tpot) / peak_bw
        mfu = 100 * (batch_size * model.estimate_decode_flops(context_mid) / tpot) / peak_flops
        print(f"{batch_size:>6} {res['ttft'] * 1e3:>9.1f} {tpot * 1e3:>9.2f} {tok_per_sec:>10,.0f} {mbu:>7.1f} {mfu:>7.2f} "
              f"{res['peak_vram'] / 2**30:>9.2f} {len(steps):>6}")
        payload["sweep"].append({"batch_size": batch_size, "ttft_sec": round(res["ttft"], 6), "tpot_sec": round(tpot, 6),
                                 "tok_per_sec": round(tok_per_sec, 1), "mbu_percent": round(mbu, 2), "mfu_percent": round(mfu, 4),
                                 "mbu_streamed_percent": round(mbu_streamed, 2),
                                 "mfu_fp8_percent": round(mfu * peak_flops / PEAK_FP8_FLOPS, 4),
                                 "peak_vram_bytes": res["peak_vram"], "decode_steps": len(steps)})
    print("-" * len(header))
    print(json.dumps(payload))


if __name__ == "__main__":
    main()
