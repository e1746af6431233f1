"""Decode throughput of the FP8 + KV-cache path on one MI355X, at the headline shape.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the headline decode configuration, whatever K and W are): nanochat d26 (n_embd 1664, 13 heads, head_dim 128,
26 layers, vocab 32768, window pattern SSSL), bf16 weights with FP8 linears, random init seed 2; one prompt of 1792 random
token ids is prefilled at batch 1, the KV cache is replicated to 64 rows, and 256 greedy tokens are decoded through
Engine.generate, which brings the context to 2048.  A "step" is one iteration of that loop: sample for all 64 rows + one
GPT.forward(ids[64,1], kv_cache).  Of the 256 steps the first W are warm-up, the LAST K are the timed ones (they end at
context 2048), the P before them carry a HIP event pair around every kernel launch (the roofline figures), and whatever lies
between warm-up and those runs untimed; the defaults 8 + 16 + 232 leave nothing in between.

One JSON line is printed with tokens/s, the roofline of the dominant kernel (decode attention, HBM bound), the rate of every
decode linear against the HBM peak, the same run with every layer reading the whole context (window pattern L), FP8 GEMM rates
at the isolated Float8Linear shapes, and a CPU baseline (the CPU oracle, a port of the reference's CPU behaviour, timed on this
box's host cores on bounded samples of the decode configurations and of the isolated GEMM shapes).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12
FP8_PEAK = 5.0e15
D26 = dict(sequence_len=2048, vocab_size=32768, n_layer=26, n_head=13, n_kv_head=13, n_embd=1664, window_pattern="SSSL")
BATCH = 64
CONTEXT = 2048
PROMPT_TOKENS = 1792
NEW_TOKENS = CONTEXT - PROMPT_TOKENS      # 256


class RangeTokenizer:
    """Engine needs four tokenizer methods; specials are placed outside the vocabulary so that random
    greedy decoding never terminates a row early."""

    def encode_special(self, s):
        return 1 << 30

    def get_bos_token_id(self):
        return (1 << 30) + 1

    def encode(self, s, prepend=None):
        return []

    def decode(self, tokens):
        return ""


def build_model(device, seed=2):
    """Random init of the d26 architecture directly on the GPU, bf16 weights with FP8 linears."""
    from nanochat_amd.gpt import GPTConfig
    from nanochat_amd.synthetic import random_init_model
    return random_init_model(GPTConfig(**D26), device, seed)


def attention_bytes_per_step(model, batch, context):
    """Algorithmic KV bytes one decode step reads at this context: per layer B * 2 * Hkv * D * 2 bytes
    per visible key, min(context, window + 1) visible keys."""
    cfg = model.config
    per_key = batch * 2 * cfg.n_kv_head * 128 * 2
    return sum(per_key * min(context, w + 1) for w, _ in model.window_sizes)


def read_profile(lib, cls):
    ms, units, n = C.c_double(), C.c_double(), C.c_int64()
    rc = lib.nc_profile_read(cls, C.byref(ms), C.byref(units), C.byref(n))
    assert rc == 0
    return ms.value, units.value, n.value


def gemm_rates(device, library_gemm=False):
    """FP8 GEMM TFLOP/s at the isolated Float8Linear shapes (M=8192), HIP events around 100 back-to-back launches.  With library_gemm, the
    ROCm library GEMM behind torch._scaled_mm (the reference's own call, nanochat/fp8.py:143-153) is timed on the same operands
    beside it, torch events around the same 60 + 100 launches."""
    from nanochat_amd import _lib, ops
    lib = _lib.lib()
    out = {}
    g = torch.Generator(device=device).manual_seed(0)
    for K, N in [(1664, 4992), (1664, 1664), (1664, 6656), (6656, 1664)]:
        M = 8192
        a = torch.randn(M, K, device=device, generator=g)
        a = (a * torch.where(torch.rand(M, K, device=device, generator=g) < 1e-3, 20.0, 1.0)).bfloat16()   # 0.1 % of the entries x 20
        w = ((torch.rand(N, K, device=device, generator=g) * 2 - 1) * (3.0 / K) ** 0.5).bfloat16()
        a8, ia, _ = ops.fp8_quantize(a)
        w8, iw, _ = ops.fp8_quantize(w)
        iw = iw.reshape(1)
        res = torch.empty(M, N, dtype=torch.bfloat16, device=device)
        def timed(fn, warm=30, n=50):
            # one event pair around n back-to-back launches: the per-launch figure carries the launch gaps, not the events
            for _ in range(warm):
                fn()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(n):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3 / n
        # 60 untimed launches first: enough back-to-back work for the clocks to settle
        fwd_us = timed(lambda: ops.fp8_gemm(a8, w8, ia, iw, out=res), warm=60, n=100)
        flops = 2.0 * M * N * K
        # quantize (amax + convert) of the activation, 3 bytes per element algorithmic, over a ring of distinct tensors larger
        # than the 256 MB memory-side cache: every pass reads its tensor from HBM, as a Float8Linear in a model does
        ring = [a] + [a.clone() for _ in range((320 << 20) // (a.numel() * 2) + 1)]
        for t in ring:
            ops.fp8_quantize(t)
        torch.cuda.synchronize()
        lib.nc_profile_enable(1)
        for i in range(max(20, 2 * len(ring))):
            ops.fp8_quantize(ring[i % len(ring)])
        torch.cuda.synchronize()
        qms, qbytes, qn = read_profile(lib, 2)
        lib.nc_profile_enable(0)
        quantize_ring_mb = len(ring) * a.numel() * 2 >> 20
        del ring
        tf = flops / (fwd_us * 1e-6) / 1e12
        # the matrix pipe's own ceiling on this shape's activation bytes: pure MFMA, no memory traffic (power-managed clock)
        ceil = mfma_ceiling(device, a8.view(torch.uint8), iters=12000)["these_operands"]
        out[f"K{K}_N{N}"] = {"us": round(fwd_us, 2), "tflops": round(tf, 1), "frac_fp8_peak": round(tf * 1e12 / FP8_PEAK, 4),
                             "mfma_only_pflops_on_these_operands": ceil["pflops"], "mfma_only_clock_ghz": ceil["shader_clock_ghz"],
                             "frac_of_mfma_only_rate": round(tf / 1e3 / ceil["pflops"], 4),
                             "quantize_us": round(qms / qn * 1e3, 2),
                             "quantize_gbps": round(qbytes / (qms * 1e-3) / 1e9, 1),
                             "quantize_frac_hbm_peak": round(qbytes / (qms * 1e-3) / HBM_PEAK, 4),
                             "quantize_distinct_input_mb": quantize_ring_mb}
        # the two backward GEMMs of the same layer (nanochat/fp8.py:156-192): e5m2 gradient x e4m3 saved operands
        go = (torch.randn(M, N, device=device, generator=g) * 1e-3).bfloat16()

        # what Float8Linear does under autograd: the output gradient quantized to e5m2 once, written as [M,N] and [N,M] by the same
        # pass; the input's transposed payload saved by the forward's quantization; the transposed weight kept with the cached weight
        go8, goT, igo, _ = ops.fp8_quantize_transposed(go, fp8_dtype=torch.float8_e5m2)
        _, xT, _, _ = ops.fp8_quantize_transposed(a)
        wT = ops.fp8_transpose(w8)
        gi = torch.empty(M, K, dtype=torch.bfloat16, device=device)
        gw = torch.empty(N, K, dtype=torch.bfloat16, device=device)
        dx_us = timed(lambda: ops.fp8_gemm_grad(go8, wT, igo, iw, out=gi))
        dw_us = timed(lambda: ops.fp8_gemm_grad(goT, xT, igo, ia, out=gw))
        # over rings of distinct tensors larger than the memory-side cache, like the forward's quantize figure
        go_ring = [go] + [go.clone() for _ in range((320 << 20) // (go.numel() * 2) + 1)]
        a_ring = [a] + [a.clone() for _ in range((320 << 20) // (a.numel() * 2) + 1)]
        ring_i = [0]

        def next_of(ring):
            ring_i[0] += 1
            return ring[ring_i[0] % len(ring)]
        prep_us = timed(lambda: ops.fp8_quantize_transposed(next_of(go_ring), fp8_dtype=torch.float8_e5m2), warm=len(go_ring), n=2 * len(go_ring))
        fwd_q_us = timed(lambda: ops.fp8_quantize_transposed(next_of(a_ring)), warm=len(a_ring), n=2 * len(a_ring))
        old_prep_us = timed(lambda: (ops.fp8_quantize(next_of(go_ring), fp8_dtype=torch.float8_e5m2), ops.fp8_transpose(w8), ops.fp8_transpose(go8),
                                     ops.fp8_transpose(a8)), warm=len(go_ring), n=2 * len(go_ring))
        del go_ring, a_ring
        out[f"K{K}_N{N}"]["backward"] = {"grad_input_us": round(dx_us, 2), "grad_weight_us": round(dw_us, 2),
                                         "grad_input_tflops": round(2.0 * M * N * K / dx_us / 1e6, 1),
                                         "grad_weight_tflops": round(2.0 * M * N * K / dw_us / 1e6, 1),
                                         "quantize_and_transposes_us": round(prep_us, 2),
                                         "quantize_and_transposes_over_gemms": round(prep_us / (dx_us + dw_us), 3),
                                         "forward_quantize_with_transposed_copy_us": round(fwd_q_us, 2),
                                         "separate_quantize_and_three_transposes_us": round(old_prep_us, 2)}
        if library_gemm:
            sa, sw = ia.reshape(()).float(), iw.reshape(()).float()
            a8t, w8t = a8.view(torch.float8_e4m3fn), w8.view(torch.float8_e4m3fn).t()

            def call():
                return torch._scaled_mm(a8t, w8t, scale_a=sa, scale_b=sw, out_dtype=torch.bfloat16, use_fast_accum=True)
            for _ in range(60):
                ref = call()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(100):
                call()
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 10.0
            out[f"K{K}_N{N}"]["library_us"] = round(us, 2)
            out[f"K{K}_N{N}"]["library_tflops"] = round(2.0 * M * N * K / us / 1e6, 1)
            out[f"K{K}_N{N}"]["rel_l2_vs_library"] = float(((res.float() - ref.float()).norm() / ref.float().norm()).item())
    return out


def mfma_ceiling(device, operands=None, iters=30000):
    """What the fp8 matrix cores sustain with nothing else running (nc_probe_fp8_mfma_ceiling): PFLOP/s and shader clock on all-zero
    operands (the published peak) and on the given e4m3 bytes.  Two launches each; the second, on a warm and settled part, counts."""
    from nanochat_amd import _lib
    lib = _lib.lib()
    clocks = torch.zeros(8, dtype=torch.int64, device=device)
    flops = C.c_double()
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for name, buf in (("zero_operands", None), ("these_operands", operands)):
        if name == "these_operands" and buf is None:
            continue
        for _ in range(2):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(lib.nc_probe_fp8_mfma_ceiling(C.c_void_p(buf.data_ptr()) if buf is not None else None,
                                                     buf.numel() * buf.element_size() if buf is not None else 0, iters,
                                                     C.c_void_p(clocks.data_ptr()), C.byref(flops), stream))
            e1.record()
            torch.cuda.synchronize()
        ms = e0.elapsed_time(e1)
        ck = clocks.tolist()
        out[name] = {"pflops": round(flops.value / (ms * 1e-3) / 1e15, 3), "ms": round(ms, 2),
                     "shader_clock_ghz": round(ck[0] / (ck[1] * 10.0), 3) if ck[1] else None}
    return out


def stream_read_floor(device, lib, sizes, reps=12):
    """What a kernel that only reads reaches here (nc_probe_hbm_read: 16-byte non-temporal loads, nothing stored), at the byte counts of
    the decode attention launches: microseconds per launch, launch and ramp included.  Every repetition reads another region of a
    2 GiB buffer, so nothing comes from the 256 MB last-level cache.  Returns {bytes: mean microseconds of the kernel itself}."""
    from nanochat_amd import _lib
    total = 2 << 30
    buf = torch.empty(total, dtype=torch.uint8, device=device)
    buf.fill_(1)
    stream = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    out = {}
    for size in sizes:
        size = min(int(size), total // 2) // 4096 * 4096
        regions = max(2, total // size)
        read = C.c_int64()
        for r in range(reps + 2):
            if r == 2:
                torch.cuda.synchronize()
                lib.nc_profile_enable(1)             # the launches from here on carry their own event pair (kernel begin / end)
            off = (r % regions) * size
            _lib.check(lib.nc_probe_hbm_read(C.c_void_p(buf.data_ptr() + off), size, C.byref(read), stream))
        torch.cuda.synchronize()
        ms, units, n = C.c_double(), C.c_double(), C.c_int64()
        assert lib.nc_profile_read(5, C.byref(ms), C.byref(units), C.byref(n)) == 0 and n.value == reps
        lib.nc_profile_enable(0)
        out[read.value] = ms.value * 1e3 / reps
    del buf
    return out


def cpu_gemm_baseline(cores, budget_s=6.0):
    """The reference's own CPU call for the isolated Float8Linear shapes (torch._scaled_mm on e4m3 operands, nanochat/fp8.py:143-153)
    and the fp8-emulated fp32 matmul beside it, on a row sample of M (the work is linear in M): GFLOP/s per shape."""
    from oracle import fp8_ref
    torch.set_num_threads(cores)
    out = {}
    g = torch.Generator().manual_seed(0)
    for K, N in [(1664, 4992), (1664, 1664), (1664, 6656), (6656, 1664)]:
        M = 512                                   # of the 8192 rows
        a = torch.randn(M, K, generator=g).bfloat16()
        w = ((torch.rand(N, K, generator=g) * 2 - 1) * (3.0 / K) ** 0.5).bfloat16()
        a8, ia, _ = fp8_ref.to_fp8(a)
        w8, iw, _ = fp8_ref.to_fp8(w)
        rec = {}
        for name, fn, rows in (("emulated_fp32_matmul", fp8_ref.scaled_mm_emulated, M), ("torch_scaled_mm", fp8_ref.scaled_mm_library, 16)):
            fn(a8[:rows], w8, ia, iw)
            n, t0 = 0, time.time()
            while n < 1 or (time.time() - t0 < budget_s / 8 and n < 20):
                fn(a8[:rows], w8, ia, iw)
                n += 1
            rec[name + "_gflops"] = round(2.0 * rows * N * K * n / (time.time() - t0) / 1e9, 2)
            rec[name + "_rows_timed"] = rows
        out[f"K{K}_N{N}"] = rec
    return out


def cpu_decode_leg(cfg_kwargs, seed, batch, ctx, max_steps, budget_s, cores):
    """Decode steps of the CPU oracle at one configuration: bf16 with fp8-emulated linears, weights re-quantized on every call as
    the reference does (fp8.py:136), on a cache filled with random keys and values (no CPU prefill is paid for)."""
    from oracle import decode_ref, gpt_ref
    torch.set_num_threads(cores)
    cfg = gpt_ref.GPTConfig(**cfg_kwargs)
    t0 = time.time()
    g = torch.Generator().manual_seed(seed)
    E, L, V, H, Hkv = cfg.n_embd, cfg.n_layer, cfg.vocab_size, cfg.n_head, cfg.n_kv_head
    s = 3 ** 0.5 * E ** -0.5
    p = {}

    # one random matrix per shape, cloned per layer: distinct memory (no cache reuse across layers) without
    # paying the host RNG for every element; timing does not depend on the values
    def u(*shape, a):
        return (torch.rand(*shape, generator=g) * 2 * a - a).bfloat16()
    w_q, w_kv, w_o = u(H * 128, E, a=s), u(Hkv * 128, E, a=s), u(E, H * 128, a=s)
    w_fc, w_pr, w_ve = u(4 * E, E, a=0.4 * s), u(E, 4 * E, a=0.5 * s), u(V, Hkv * 128, a=s)
    p["transformer.wte.weight"] = torch.randn(V, E, generator=g).bfloat16()
    p["lm_head.weight"] = (torch.randn(V, E, generator=g) * 0.03).bfloat16()
    for i in range(L):
        pre = f"transformer.h.{i}."
        p[pre + "attn.c_q.weight"] = w_q.clone()
        p[pre + "attn.c_k.weight"] = w_kv.clone()
        p[pre + "attn.c_v.weight"] = w_kv.clone()
        p[pre + "attn.c_proj.weight"] = w_o.clone()
        p[pre + "mlp.c_fc.weight"] = w_fc.clone()
        p[pre + "mlp.c_proj.weight"] = w_pr.clone()
        if gpt_ref.has_ve(i, L):
            p[f"value_embeds.{i}.weight"] = w_ve.clone()
            p[pre + "attn.ve_gate.weight"] = torch.rand(Hkv, 12, generator=g) - 0.5
    p["resid_lambdas"] = torch.linspace(1.15, 1.05, L)
    p["x0_lambdas"] = torch.linspace(0.20, 0.05, L)
    p["smear_lambda"] = torch.full((1,), 0.35)
    p["backout_lambda"] = torch.full((1,), 0.2)
    p["smear_gate.weight"] = torch.rand(1, 24, generator=g) - 0.5
    rt = gpt_ref.Runtime(cfg, p, compute_dtype=torch.bfloat16, fp8=True, cache_weights=False)
    cache = decode_ref.new_cache(cfg, batch, ctx + max_steps, torch.bfloat16)
    kblk = (torch.randn(1, 1, ctx, Hkv, 128, generator=g) * 1.2).bfloat16()
    vblk = (torch.randn(1, 1, ctx, Hkv, 128, generator=g) * 0.5).bfloat16()
    cache.k_cache[:, :, :ctx] = kblk
    cache.v_cache[:, :, :ctx] = vblk
    cache.cache_seqlens.fill_(ctx)
    cache.prev_embedding = torch.randn(batch, 1, E, generator=g).bfloat16()
    setup_s = time.time() - t0
    ids = torch.randint(0, V, (batch, 1), generator=g)
    steps, spent = 0, 0.0
    while steps < 1 or (spent < budget_s and steps < max_steps):
        t1 = time.time()
        logits = gpt_ref.forward(rt, ids, cache)
        ids = logits[:, -1].argmax(-1, keepdim=True)
        spent += time.time() - t1
        steps += 1
    return {"tokens_per_s": round(batch * steps / spent, 3), "s_per_step": round(spent / steps, 4), "steps_timed": steps,
            "batch": batch, "context": ctx, "setup_s_not_timed": round(setup_s, 1)}


def cpu_config1_leg(cores):
    """BASELINE configs[0] in full, the way scripts/infer_bench.py:73-79,207-216 times a run: the d4 model in fp32 on the CPU, the
    repository's init (seed 0), batch 1, a 32-token prompt, 64 greedy tokens; tokens/s over prefill + decode."""
    from oracle import decode_ref, gpt_ref
    torch.set_num_threads(cores)
    cfg = gpt_ref.GPTConfig(sequence_len=2048, vocab_size=32768, n_layer=4, n_head=2, n_kv_head=2, n_embd=256)
    params = gpt_ref.init_params(cfg, seed=0, compute_dtype=torch.float32)
    rt = gpt_ref.Runtime(cfg, params, compute_dtype=torch.float32, fp8=False)
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, 32768, (32,), generator=g).tolist()
    decode_ref.generate(rt, prompt, 1, 4, temperature=0.0)            # one short run first (allocator, thread pool)
    t0 = time.time()
    out, _ = decode_ref.generate(rt, prompt, 1, 64, temperature=0.0)
    dt = time.time() - t0
    return {"tokens_per_s": round(len(out) / dt, 2), "seconds": round(dt, 3), "new_tokens": len(out), "prompt_tokens": 32,
            "batch": 1, "dtype": "fp32, plain linears"}


def cpu_baseline():
    """The CPU oracle on this box's host cores, bounded samples: the headline configuration (configs[3]: d26, 64 rows, context
    1792; up to 4 decode steps), configs[2] (d20, 8 rows, context 512; the first 8 decode steps), configs[0] in full (d4 fp32, one
    row, 32-token prompt + 64 greedy tokens), and row samples of the isolated GEMM shapes (configs[1])."""
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
    c4 = cpu_decode_leg(D26 | {"window_pattern": "SSSL"}, 2, BATCH, PROMPT_TOKENS, 4, 12.0, cores)
    d20 = dict(sequence_len=2048, vocab_size=32768, n_layer=20, n_head=10, n_kv_head=10, n_embd=1280, window_pattern="SSSL")
    c3 = cpu_decode_leg(d20, 1, 8, 512, 8, 8.0, cores)
    c1 = cpu_config1_leg(cores)
    return {"value": c4["tokens_per_s"], "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{c4['steps_timed']} decode step(s) of the CPU oracle at d26, 64 rows, context {PROMPT_TOKENS} (random-filled cache), "
                      f"bf16 + fp8-emulated linears with per-call weight quantization as in the reference; setup "
                      f"{c4['setup_s_not_timed']:.0f}s not timed",
            "s_per_step": c4["s_per_step"],
            "config3_d20_b8_ctx512": c3 | {"sample": f"first {c3['steps_timed']} decode steps, greedy, random-filled cache"},
            "config1_d4_fp32_b1": c1 | {"sample": "full: 32-token prompt + 64 greedy tokens through the oracle's generate loop"},
            "fp8_gemm_m8192": cpu_gemm_baseline(cores)}


def attention_sources_digest():
    """SHA-256 over the sources of the decode-attention kernel: ties a counter measurement to the code it was taken on."""
    import hashlib
    h = hashlib.sha256()
    for f in ("nc_attention.hip", "nc_rope.h", "nc_common.h"):
        h.update(open(os.path.join(ROOT, "nanochat_amd", "csrc", f), "rb").read())
    return h.hexdigest()


def measured_traffic():
    """HBM bytes per attention launch from the hardware counters (FETCH_SIZE + WRITE_SIZE of rocprofv3 --pmc runs of this
    script, scaled by what the same counters read for the --copy-probe-mib pass).  The counters cannot be collected from
    inside this process, so the figure is read from the summary committed next to the profiles, which names the kernel
    sources it was measured on: (bytes, note); bytes is None if the summary is absent or was taken on other sources."""
    path = os.path.join(ROOT, "profiles", "attn_partial_d26_b64_traffic.json")
    try:
        with open(path) as f:
            rec = json.load(f)
        if rec.get("kernel_sources_sha256") != attention_sources_digest():
            return None, "profiles/attn_partial_d26_b64_traffic.json was measured on other kernel sources than this tree holds"
        return rec["hbm_bytes_per_launch"], "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script on these kernel sources (profiles/)"
    except (OSError, KeyError, ValueError):
        return None, "no counter summary under profiles/"


def set_window_pattern(model, pattern):
    """Switch the sliding-window pattern of a built model: the weights do not depend on it, the per-layer windows of the plan do."""
    from nanochat_amd.gpt import compute_window_sizes
    model.config.window_pattern = pattern
    model.window_sizes = compute_window_sizes(model.config)
    model.invalidate_plan()


def run_decode(model, lib, K, W, P, pattern, share_prompt_reads=False):
    """The headline protocol on `model` with the given window pattern: 1792-token prompt, 64 rows, 256 greedy tokens; W warm-up steps,
    untimed steps, P steps with a HIP event pair around every kernel launch, and the last K steps timed.  Returns the figures."""
    from nanochat_amd.engine import Engine
    set_window_pattern(model, pattern)
    filler = NEW_TOKENS - (W + P + K)
    engine = Engine(model, RangeTokenizer())
    g = torch.Generator().manual_seed(2)
    prompt = torch.randint(0, D26["vocab_size"], (PROMPT_TOKENS,), generator=g).tolist()

    # one-off work (FP8 weight quantization of the plan, workspace allocation) is kept out of the time to first token
    for _ in engine.generate(prompt[:64], num_samples=2, max_tokens=2, temperature=0.0):
        pass
    torch.cuda.synchronize()
    gen = engine.generate(prompt, num_samples=BATCH, max_tokens=NEW_TOKENS + 1, temperature=0.0, share_prompt_reads=share_prompt_reads)
    t_pre = time.perf_counter()
    next(gen)                                  # prefill + cache replication + first sample + first forward
    torch.cuda.synchronize()
    ttft = time.perf_counter() - t_pre
    for _ in range(W - 1 + filler):
        next(gen)
    torch.cuda.synchronize()
    first_profiled = PROMPT_TOKENS + W + filler         # cache length the first profiled forward starts from

    # ---- kernel-level timing, HIP events on the launch stream, same process and state, right in front of the timed steps
    lib.nc_profile_enable(1)
    for _ in range(P):
        next(gen)
    torch.cuda.synchronize()
    prof = {c: read_profile(lib, c) for c in range(5)}
    E, H, Hkv, V = D26["n_embd"], D26["n_head"], D26["n_kv_head"], D26["vocab_size"]
    linears = {}
    for name, (N, Kd) in (("qkv", ((H + 2 * Hkv) * 128, E)), ("attn_c_proj", (E, H * 128)), ("c_fc", (4 * E, E)), ("mlp_c_proj", (E, 4 * E)),
                          ("lm_head", (V, E))):
        ms, units, n = C.c_double(), C.c_double(), C.c_int64()
        assert lib.nc_profile_read_gemm(N, Kd, C.byref(ms), C.byref(units), C.byref(n)) == 0
        if n.value:
            us = ms.value * 1e3 / n.value
            # a decode linear streams its e4m3 weight once: N * K bytes (the 64 activation rows are L2 traffic)
            linears[name] = {"weight_bytes": N * Kd, "launches_timed": n.value, "avg_launch_us": round(us, 2),
                             "gbps": round(N * Kd / us / 1e3, 1), "frac_hbm_peak": round(N * Kd / (us * 1e-6) / HBM_PEAK, 4)}
    lib.nc_profile_enable(0)

    step_times = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(K):
        t1 = time.perf_counter()
        next(gen)
        step_times.append(time.perf_counter() - t1)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    gen.close()
    del gen, engine
    att_ms, _, att_n = prof[0]
    # the P profiled forwards ran at cache lengths first_profiled .. first_profiled + P - 1 (each then sees one more key: itself)
    launches_per_step = model.config.n_layer
    att_bytes_step = sum(attention_bytes_per_step(model, BATCH, first_profiled + j + 1) for j in range(P)) / P
    att_avg_s = att_ms * 1e-3 / att_n
    att_bytes_launch = att_bytes_step / launches_per_step
    weight_bytes_step = sum(v["weight_bytes"] * (1 if k == "lm_head" else model.config.n_layer) for k, v in linears.items())
    return {"tok_per_s": BATCH * K / elapsed, "ms_per_step": elapsed / K * 1e3, "ttft": ttft,
            "tpot_ms_median": sorted(step_times)[len(step_times) // 2] * 1e3,
            "att_bytes_launch": att_bytes_launch, "att_avg_s": att_avg_s, "att_n": att_n, "att_bytes_step": att_bytes_step,
            "kernel_ms_per_step": {name: round(prof[c][0] / P, 3) for c, name in enumerate(["attention", "fp8_gemm", "quantize", "rows", "sampler"])},
            "linears": linears, "weight_bytes_step": weight_bytes_step,
            "profiled_steps_context": [first_profiled + 1, first_profiled + P], "filler": filler}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=232)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm", action="store_true")
    ap.add_argument("--no-pattern-l", action="store_true", help="skip the second run with every layer reading the whole context")
    ap.add_argument("--no-stream-probe", action="store_true", help="skip the read-only kernel timed beside the attention launches")
    ap.add_argument("--no-shared-prompt", action="store_true", help="skip the extra run that reads the replicated prompt once for all rows")
    ap.add_argument("--library-gemm", action="store_true", help="also time torch._scaled_mm on the M=8192 GEMM operands")
    ap.add_argument("--profile-steps", type=int, default=16)
    ap.add_argument("--window-pattern", default="SSSL",
                    help="sliding-window pattern of the layers (the headline number is SSSL; L makes every layer read the whole context)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="after the decode steps, run an elementwise pass that reads and writes this many MiB "
                         "(a kernel of known traffic to scale hardware byte counters with)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (decode would shard by batch row, one independent copy per GPU). "
              "Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    from nanochat_amd import _lib
    lib = _lib.lib()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    K, W = args.steps, max(1, args.warmup)
    assert 1 <= K and W + K + 1 <= NEW_TOKENS, f"warmup + steps must leave at least one of the {NEW_TOKENS} new tokens for the profiled steps"
    P = max(1, min(args.profile_steps, NEW_TOKENS - W - K))       # what the 256 new tokens leave room for
    model = build_model(device)
    r = run_decode(model, lib, K, W, P, args.window_pattern)
    if args.copy_probe_mib > 0:
        n = args.copy_probe_mib * (1 << 20) // 2
        src = torch.ones(n, dtype=torch.bfloat16, device=device)
        dst = torch.empty_like(src)
        for _ in range(4):
            torch.mul(src, 1.0, out=dst)       # reads n*2 bytes, writes n*2 bytes
        torch.cuda.synchronize()
        del src, dst
    achieved = r["att_bytes_launch"] / r["att_avg_s"]
    traffic, traffic_note = measured_traffic() if args.window_pattern == "SSSL" else (None, "counter summary exists for window pattern SSSL only")

    result = {
        "metric": "decode tokens/sec @ d26 bs64 ctx2048",
        "value": round(r["tok_per_s"], 1),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": args.warmup,
        "ms_per_step": round(r["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3 x fp8_e4m3 -> fp32 acc (linears), bf16 (KV cache, activations)",
        "data": "synthetic: random token ids, random-init weights of the d26 architecture (seed 2)",
        "config": {"workload": f"nanochat d26 decode (BASELINE configs[3]), batch 64, prompt {PROMPT_TOKENS} tokens, {NEW_TOKENS} new tokens, "
                               f"timed: the last {K} steps, context {CONTEXT - K}->{CONTEXT}, greedy, window pattern {args.window_pattern}, "
                               "Engine.generate loop (sample + GPT.forward with KV cache per step)",
                   "batch": BATCH, "context_end": CONTEXT, "prompt_tokens": PROMPT_TOKENS, "new_tokens": NEW_TOKENS,
                   "untimed_steps_before_the_profiled_ones": W + r["filler"], "profiled_steps": P,
                   "profiled_steps_context": r["profiled_steps_context"]},
        "tpot_ms_median": round(r["tpot_ms_median"], 4),
        "ttft_s": round(r["ttft"], 3),
        "roofline": {"bound": "hbm", "kernel": "attn_partial_kernel (+combine) per layer launch",
                     "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4),
                     "traffic": traffic, "traffic_source": traffic_note,
                     "bytes_per_launch": int(r["att_bytes_launch"]), "avg_launch_us": round(r["att_avg_s"] * 1e6, 2),
                     "launches_timed": r["att_n"]},
        "kernel_ms_per_step": r["kernel_ms_per_step"],
        # the weight-streaming linears of the decode step against the HBM peak (HIP events around each launch, in-step)
        "decode_linears": r["linears"],
        # the reference's MBU numerator with the bytes really streamed: e4m3 weights + KV read at the profiled context
        "step_bytes": {"weights_e4m3": r["weight_bytes_step"], "kv_read": int(r["att_bytes_step"]),
                       "frac_hbm_peak_whole_step": round((r["weight_bytes_step"] + r["att_bytes_step"]) / (r["ms_per_step"] * 1e-3) / HBM_PEAK, 4)},
    }
    if not args.no_stream_probe:
        # beside the published peak: the duration of a read-only kernel over the bytes of a window layer's and a full-context layer's
        # launch; between the two sizes the time is linear in the bytes, which prices the average launch (a mix of both kinds)
        b_small = BATCH * 2 * model.config.n_kv_head * 128 * 2 * 513
        b_large = BATCH * 2 * model.config.n_kv_head * 128 * 2 * CONTEXT
        torch.cuda.empty_cache()
        fl = stream_read_floor(device, lib, (b_small, b_large))
        (s0, t0), (s1, t1) = sorted(fl.items())
        per_byte = (t1 - t0) / (s1 - s0)
        floor_us = t0 + (r["att_bytes_launch"] - s0) * per_byte
        result["roofline"]["read_only_kernel"] = {
            "bytes": [s0, s1], "us": [round(t0, 2), round(t1, 2)], "GBps": [round(s0 / t0 / 1e3, 1), round(s1 / t1 / 1e3, 1)],
            "us_for_bytes_per_launch": round(floor_us, 2), "frac_of_it": round(floor_us / (r["att_avg_s"] * 1e6), 4),
            "note": "nc_probe_hbm_read, launches that carry their own event pair like the attention launches, over regions of a 2 GiB buffer: what reading the same bytes once costs "
                    "a kernel that does nothing else; frac_of_it = that time / avg_launch_us"}
    if args.window_pattern == "SSSL" and not args.no_pattern_l:
        # the same configuration with every layer reading the whole context (22.7 GB of KV per step at context 2048): the case
        # that is bound by KV reads alone; a shorter timed window, same prompt, same 256 new tokens
        KL = min(K, 64)
        PL = max(1, min(P, 8))
        torch.cuda.empty_cache()
        rl = run_decode(model, lib, KL, W, PL, "L")
        ach_l = rl["att_bytes_launch"] / rl["att_avg_s"]
        result["window_pattern_L"] = {
            "value": round(rl["tok_per_s"], 1), "unit": "tokens/s", "ms_per_step": round(rl["ms_per_step"], 4), "steps": KL,
            "workload": f"same model, prompt and batch with window pattern L; timed: the last {KL} of the {NEW_TOKENS} steps",
            "roofline": {"bound": "hbm", "achieved": round(ach_l / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                         "frac": round(ach_l / HBM_PEAK, 4), "bytes_per_launch": int(rl["att_bytes_launch"]),
                         "avg_launch_us": round(rl["att_avg_s"] * 1e6, 2), "launches_timed": rl["att_n"]},
            "kernel_ms_per_step": rl["kernel_ms_per_step"],
            "step_bytes": {"weights_e4m3": rl["weight_bytes_step"], "kv_read": int(rl["att_bytes_step"]),
                           "frac_hbm_peak_whole_step": round((rl["weight_bytes_step"] + rl["att_bytes_step"]) / (rl["ms_per_step"] * 1e-3) / HBM_PEAK, 4)}}
    if args.window_pattern == "SSSL" and not args.no_shared_prompt:
        # Not the headline: the same run with Engine.generate(share_prompt_reads=True).  The 64 rows are copies of one prompt
        # (that is how Engine.generate builds a batch), so the full-context layers can read the prompt's keys and values once for
        # all rows on the matrix cores and stream per row only the tokens decoded since; `value` above reads every row's copy.
        torch.cuda.empty_cache()
        rs = run_decode(model, lib, K, W, P, "SSSL", share_prompt_reads=True)
        result["shared_prompt_reads"] = {
            "value": round(rs["tok_per_s"], 1), "unit": "tokens/s", "ms_per_step": round(rs["ms_per_step"], 4), "steps": K,
            "workload": "same model, prompt, batch and window pattern; the full-context layers read the replicated prompt once for all rows "
                        "(Engine.generate(share_prompt_reads=True), off by default)",
            "kernel_ms_per_step": rs["kernel_ms_per_step"], "tpot_ms_median": round(rs["tpot_ms_median"], 4)}
    if not args.no_gemm:
        result["fp8_gemm_m8192"] = gemm_rates(device, args.library_gemm)
        # the published 5.0 PFLOP/s is what all-zero operands sustain; random e4m3 bytes settle at a lower clock
        rnd = torch.randint(0, 127, (1 << 20,), dtype=torch.uint8, device=device) | (torch.randint(0, 2, (1 << 20,), dtype=torch.uint8, device=device) << 7)
        result["fp8_mfma_only"] = mfma_ceiling(device, rnd)
        result["fp8_mfma_only"]["note"] = ("pure v_mfma_f32_16x16x128_f8f6f4 loop on every SIMD, no memory or LDS traffic: the rate the part's "
                                           "power management sustains; these_operands = uniformly random finite e4m3 bytes")
    del model
    torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
