"""GPU parity of the whole path: GPT.forward(idx, kv_cache=...) / Engine.generate on the HIP kernels
against the CPU oracle on the same seeded weights and inputs.

Bars.
  * Repository init (the reference's own init_weights: zero-initialised projections, lm_head std 0.001 -- the weights the
    stated tolerance is quoted on): logits within 1e-2 abs of the oracle, the 64 greedy ids identical to the
    oracle's (asserted strictly on the fixed seed).
  * "Trained-like" init (non-zero projections, O(1) logits, so attention / MLP / smear / KV cache all
    matter): dynamic tensorwise FP8 re-quantizes every activation, which amplifies any last-bit
    difference to the fp8 noise level within a few layers.  The oracle itself moves by rel-L2 ~4e-2
    (max ~0.1 at |logit| ~2.5) when its attention is switched between two forms the reference treats as
    equal (SDPA vs the fp32 definition; the reference's own FA3-vs-SDPA tolerance is 1e-2 on attention
    outputs).  The bar is therefore that sensitivity floor: the HIP path may be no further from the
    oracle than 1.5x the distance between those two oracle variants.  Stage-wise exactness on
    identical inputs is covered by tests/test_gpu_kernels.py and by the layer-wise test below.
"""
import hashlib
import json
import os
import sys

import pytest
import torch

from oracle import gpt_ref, decode_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"
GOLD = os.path.join(os.path.dirname(__file__), "golden")
LOGIT_TOL = 1e-2


def say(msg):
    print(f"[gpu-case] {msg}", flush=True)
    sys.stdout.flush()


def build_pair(cfg_kwargs, seed, trained_like=True):
    """(oracle runtime, product model on the GPU) sharing one set of weights."""
    from nanochat_amd.gpt import GPT, GPTConfig
    from nanochat_amd.fp8 import convert_to_float8_training, fp8_module_filter
    ocfg = gpt_ref.GPTConfig(**cfg_kwargs)
    params = gpt_ref.init_params(ocfg, seed=seed, compute_dtype=torch.bfloat16, trained_like=trained_like)
    rt = gpt_ref.Runtime(ocfg, params, compute_dtype=torch.bfloat16, fp8=True)
    with torch.device("meta"):
        model = GPT(GPTConfig(**cfg_kwargs))
    model.to_empty(device="cpu")
    model.transformer.wte.to(torch.bfloat16)
    for ve in model.value_embeds.values():
        ve.to(torch.bfloat16)
    model.load_reference_state(params)
    model.to(DEV)
    convert_to_float8_training(model, module_filter_fn=fp8_module_filter)
    return rt, model


D4 = dict(sequence_len=2048, vocab_size=32768, n_layer=4, n_head=2, n_kv_head=2, n_embd=256)
SMALL_GQA = dict(sequence_len=256, vocab_size=1024, n_layer=5, n_head=4, n_kv_head=2, n_embd=512, window_pattern="SL")
SMALL_MHA = dict(sequence_len=512, vocab_size=2048, n_layer=6, n_head=3, n_kv_head=3, n_embd=384, window_pattern="SSSL")
# batch x kv heads = 512: attention runs one workgroup per (row, kv head), unsplit, and finishes q|k|v (rotary, append) itself;
# the variant with two kv heads per workgroup needs batch x ceil(kv heads / 2) >= 384 and is covered in test_gpu_variants.py
WIDE_GQA = dict(sequence_len=128, vocab_size=1024, n_layer=3, n_head=8, n_kv_head=4, n_embd=1024, window_pattern="SL")
WIDE_MHA = dict(sequence_len=128, vocab_size=1024, n_layer=2, n_head=4, n_kv_head=4, n_embd=512, window_pattern="SL")


@pytest.fixture(scope="module")
def d4_pair():
    return build_pair(D4, seed=0, trained_like=True)


@pytest.fixture(scope="module")
def d4_repo_pair():
    return build_pair(D4, seed=0, trained_like=False)


def rel_l2(a, b):
    return ((a.float() - b.float()).norm() / b.float().norm().clamp_min(1e-30)).item()


def oracle_floor(rt, run):
    """Distance between two reference-equivalent oracle variants (SDPA attention vs the fp32 definition)
    on the computation `run(runtime) -> logits`; returns (rel_l2, max_abs, sdpa_logits, def_logits)."""
    rt_def = gpt_ref.Runtime(rt.cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    a, b = run(rt), run(rt_def)
    return rel_l2(b, a), (a - b).abs().max().item(), a, b


def bar(what, value, recorded, margin):
    """A bar written as the value observed when the test was written plus a stated margin; what this run observes is printed, so a
    drift towards the bar shows in the log before it fails."""
    print(f"[bar] {what}: observed {value:.5g} (recorded {recorded:.5g} + margin {margin:.5g} = bar {recorded + margin:.5g})")
    assert value <= recorded + margin, f"{what}: {value} exceeds {recorded} + {margin}"


def assert_within_floor(got, want_sdpa, want_def, floor_rel, floor_max, what):
    r1, r2 = rel_l2(got, want_sdpa), rel_l2(got, want_def)
    m1, m2 = (got - want_sdpa).abs().max().item(), (got - want_def).abs().max().item()
    print(f"{what}: vs SDPA-oracle rel_l2 {r1:.4f} max {m1:.4f}; vs fp32-definition oracle rel_l2 {r2:.4f} max {m2:.4f}; "
          f"oracle-vs-oracle floor rel_l2 {floor_rel:.4f} max {floor_max:.4f}")
    assert min(r1, r2) <= 1.5 * floor_rel + 1e-3, what
    assert min(m1, m2) <= 1.5 * floor_max + LOGIT_TOL, what


def test_repo_init_logits_and_greedy_ids(d4_repo_pair):
    """Repository-init weights: logits within 1e-2 abs, greedy ids identical for 64 tokens."""
    say("d4 repo init: prefill logits + 64 greedy tokens")
    rt, model = d4_repo_pair
    from nanochat_amd.engine import KVCache
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, 32768, (32,), generator=g).tolist()
    want_cols, want_logits = decode_ref.generate(rt, prompt, 1, 64, temperature=0.0, collect_logits=True)
    want_ids = [c[0] for c in want_cols]
    cache = KVCache(1, 2, 96, 128, 4, DEV, torch.bfloat16)
    logits = model.forward_last(torch.tensor([prompt]).to(DEV), kv_cache=cache).cpu()
    worst, got_ids = 0.0, []
    for t in range(64):
        worst = max(worst, (logits[0] - want_logits[t][0]).abs().max().item())
        got_ids.append(int(logits[0].argmax()))
        nxt = torch.tensor([[want_ids[t]]])                 # teacher forcing keeps every step comparable
        logits = model.forward_last(nxt.to(DEV), kv_cache=cache).cpu()
    same = sum(int(a == b) for a, b in zip(got_ids, want_ids))
    print(f"repo init: max |dlogit| over 64 steps = {worst:.6f}; greedy ids equal on {same}/64 steps")
    assert worst <= LOGIT_TOL
    # strict: on this seed all 64 ids are the oracle's; the oracle's own top-2 margin at a differing step only explains a failure
    diverged = [(t, a, b, (lambda v: (v[0] - v[1]).item())(torch.topk(want_logits[t][0], 2).values))
                for t, (a, b) in enumerate(zip(got_ids, want_ids)) if a != b]
    assert not diverged, f"greedy ids differ from the oracle's at (step, got, want, oracle top-2 margin): {diverged}"


def test_prefill_logits_match_oracle(d4_pair):
    say("d4 trained-like prefill logits")
    rt, model = d4_pair
    from nanochat_amd.engine import KVCache
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, 32768, (1, 32), generator=g)
    caches = []

    def run(r):
        c = decode_ref.new_cache(r.cfg, 1, 64, torch.bfloat16)
        caches.append(c)
        return gpt_ref.forward(r, prompt, c)
    floor_rel, floor_max, want, want_def = oracle_floor(rt, run)
    ref_cache = caches[0]
    cache = KVCache(1, 2, 64, 128, 4, DEV, torch.bfloat16)
    got = model(prompt.to(DEV), kv_cache=cache).cpu()
    assert got.shape == want.shape == (1, 32, 32768) and got.dtype == torch.float32
    assert_within_floor(got, want, want_def, floor_rel, floor_max, "prefill logits")
    assert cache.get_pos() == 32 and cache.cache_seqlens.tolist() == [32]
    # layer 0 sees identical inputs on both sides: its appended K/V must agree to the last bf16 bit or so
    k0 = (cache.k_cache[0].cpu().float() - ref_cache.k_cache[0].float()).abs()
    v0 = (cache.v_cache[0].cpu().float() - ref_cache.v_cache[0].float()).abs()
    assert k0.max().item() <= 0.04 and v0.max().item() <= 0.04 and (k0 > 0).float().mean().item() < 0.02
    assert torch.allclose(cache.prev_embedding.cpu().float(), ref_cache.prev_embedding.float(), atol=2e-2)


def test_greedy_decode_64_tokens_through_engine(d4_repo_pair):
    """Engine.generate on the GPU, greedy, 64 tokens, repository init: all 64 ids equal to the oracle's (strictly; the oracle's own
    top-2 margin at a differing step is only printed with the failure).  The trained-like counterpart, with a bound derived from the oracle's own sensitivity, is in test_gpu_variants.py."""
    from nanochat_amd.engine import Engine
    from test_engine_host import ByteTokenizer

    class Tok(ByteTokenizer):          # specials placed where random logits will not pick them by accident
        def __init__(self):
            self._special = {"<|python_start|>": 32760, "<|python_end|>": 32761, "<|output_start|>": 32762,
                             "<|output_end|>": 32763, "<|assistant_end|>": 32764, "<|bos|>": 32765}

        def get_bos_token_id(self):
            return 32765
    g = torch.Generator().manual_seed(0)
    prompt = torch.randint(0, 32768, (32,), generator=g).tolist()
    rt, model = d4_repo_pair
    say("d4 repo: greedy decode 64 tokens via Engine.generate")
    want_cols, want_logits = decode_ref.generate(rt, prompt, 1, 64, temperature=0.0, collect_logits=True)
    want_ids = [c[0] for c in want_cols]
    got_ids = []
    for column, masks in Engine(model, Tok()).generate(prompt, num_samples=1, max_tokens=64, temperature=0.0):
        got_ids.append(column[0])
        if column[0] in (32764, 32765):
            break
    first_div = next((i for i, (a, b) in enumerate(zip(got_ids, want_ids)) if a != b), len(got_ids))
    print(f"repo: greedy ids identical for the first {first_div} of {len(got_ids)} tokens")
    gap = None
    if first_div < min(len(got_ids), len(want_ids)):
        top2 = torch.topk(want_logits[first_div][0], 2).values
        gap = (top2[0] - top2[1]).item()          # the diagnostic: how close the oracle's own decision was at the first differing step
    # strict: all 64 ids identical on this seed
    assert len(got_ids) == 64 and got_ids == want_ids, f"token {first_div} differs; the oracle's top-2 margin there is {gap}"


def test_decode_logits_stepwise_teacher_forced(d4_pair):
    """Feed the SDPA-oracle's tokens to every side so each step stays comparable."""
    say("d4 trained-like decode logits, teacher forced, B=3")
    rt, model = d4_pair
    from nanochat_amd.engine import KVCache
    g = torch.Generator().manual_seed(1)
    B, P, steps = 3, 20, 24
    prompt = torch.randint(0, 32768, (B, P), generator=g)
    rt_def = gpt_ref.Runtime(rt.cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    c_sdpa = decode_ref.new_cache(rt.cfg, B, P + steps, torch.bfloat16)
    c_def = decode_ref.new_cache(rt.cfg, B, P + steps, torch.bfloat16)
    cache = KVCache(B, 2, P + steps, 128, 4, DEV, torch.bfloat16)
    seq_s, seq_d, seq_g = [], [], []
    ids = prompt
    for s in range(steps + 1):
        a = gpt_ref.forward(rt, ids, c_sdpa)[:, -1]
        b = gpt_ref.forward(rt_def, ids, c_def)[:, -1]
        c = model.forward_last(ids.to(DEV), kv_cache=cache).cpu()
        seq_s.append(a), seq_d.append(b), seq_g.append(c)
        ids = a.argmax(-1, keepdim=True)
    S, Dd, G = torch.stack(seq_s), torch.stack(seq_d), torch.stack(seq_g)
    assert_within_floor(G, S, Dd, rel_l2(Dd, S), (S - Dd).abs().max().item(), f"{steps + 1} teacher-forced steps")
    agree = (G.argmax(-1) == S.argmax(-1)).float().mean().item()
    agree_floor = (Dd.argmax(-1) == S.argmax(-1)).float().mean().item()
    print(f"argmax agreement with the SDPA oracle: HIP {agree:.2f}, fp32-definition oracle {agree_floor:.2f}")
    assert agree >= agree_floor - 0.15
    assert cache.get_pos() == P + steps


def test_reference_written_goldens(d4_pair, d4_repo_pair):
    """Against numbers the reference's own GPT produced in the authoring container (tests/golden)."""
    with open(os.path.join(GOLD, "gpt_d4_bf16_fp8.json")) as f:
        gold = json.load(f)

    def sha(t):
        t = t.detach().contiguous()
        raw = t.view(torch.int16).numpy().tobytes() if t.dtype == torch.bfloat16 else t.numpy().tobytes()
        return hashlib.sha256(raw).hexdigest()
    from nanochat_amd.engine import KVCache
    checked = 0
    for name, (rt, model) in (("repo", d4_repo_pair), ("trained_like", d4_pair)):
        say(f"d4 {name} vs reference-written goldens")
        run = gold["runs"][name]
        bad = [k for k, h in run["weight_sha256"].items() if sha(rt.p[k]) != h]
        if bad:
            print(f"{name}: this host's torch RNG does not reproduce the golden weights ({bad[:2]}); skipped")
            continue
        checked += 1
        prompt = torch.tensor([gold["prompt"]])
        cache = KVCache(1, 2, 32 + 64, 128, 4, DEV, torch.bfloat16)
        logits = model.forward_last(prompt.to(DEV), kv_cache=cache).cpu()
        # the floor: the oracle's fp32-definition variant (a form the reference treats as equal to its SDPA path, which wrote the
        # goldens) on the same tokens, measured on the same samples of every logits row
        rt_def = gpt_ref.Runtime(rt.cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
        c_def = decode_ref.new_cache(rt.cfg, 1, 32 + 64, torch.bfloat16)
        other = gpt_ref.forward(rt_def, prompt, c_def)[:, -1]
        worst, num, den, f_worst, f_num = 0.0, 0.0, 0.0, 0.0, 0.0
        for t in range(40):
            dig = run["steps"][t]["digest"]
            row, orow = logits[0], other[0]
            for pick, want in ((slice(0, 32), dig["head"]), (slice(None, None, 1021), dig["strided"]), (dig["top_idx"], dig["top_val"])):
                want = torch.tensor(want)
                worst = max(worst, (row[pick] - want).abs().max().item())
                num += (row[pick] - want).pow(2).sum().item()
                den += want.pow(2).sum().item()
                f_worst = max(f_worst, (orow[pick] - want).abs().max().item())
                f_num += (orow[pick] - want).pow(2).sum().item()
            nxt = torch.tensor([[run["greedy_ids"][t]]])          # teacher forcing with the reference's ids
            logits = model.forward_last(nxt.to(DEV), kv_cache=cache).cpu()
            other = gpt_ref.forward(rt_def, nxt, c_def)[:, -1]
        rel, f_rel = (num / den) ** 0.5, (f_num / den) ** 0.5
        print(f"{name} vs reference goldens: max |dlogit| = {worst:.5f}, rel_l2 = {rel:.4f}; the oracle's other variant: "
              f"max {f_worst:.5f}, rel_l2 {f_rel:.4f}")
        if name == "repo":
            assert worst <= LOGIT_TOL
        else:
            assert rel <= 1.5 * f_rel + 1e-3 and worst <= 1.5 * f_worst + LOGIT_TOL
    if checked == 0:
        pytest.skip("golden weights not reproducible on this host")


def test_cached_decode_equals_cache_free_forward(d4_pair):
    say("cached == cache-free")
    rt, model = d4_pair
    from nanochat_amd.engine import KVCache
    g = torch.Generator().manual_seed(2)
    seq = torch.randint(0, 32768, (2, 24), generator=g).to(DEV)
    full = model(seq)                                    # no cache: whole sequence at once
    cache = KVCache(2, 2, 32, 128, 4, DEV, torch.bfloat16)
    part = model(seq[:, :16], kv_cache=cache)
    rows = [part[:, -1]]
    for t in range(16, 24):
        rows.append(model(seq[:, t:t + 1], kv_cache=cache)[:, -1])
    stepped = torch.stack(rows, dim=1)                   # logits at positions 15..23
    # Not bit-equal: the activation scale of an FP8 linear is tensorwise over the rows of the call, so a
    # 24-token call and a 1-token call quantize differently.  The oracle does the same computation both ways; the gap it
    # shows between its two ways is the yardstick, and each way is checked against the oracle's.
    seq_c = seq.cpu()
    full_o = gpt_ref.forward(rt, seq_c, None)
    c = decode_ref.new_cache(rt.cfg, 2, 32, torch.bfloat16)
    rows_o = [gpt_ref.forward(rt, seq_c[:, :16], c)[:, -1]]
    for t in range(16, 24):
        rows_o.append(gpt_ref.forward(rt, seq_c[:, t:t + 1], c)[:, -1])
    stepped_o = torch.stack(rows_o, dim=1)
    gap_o = (stepped_o - full_o[:, 15:]).abs().max().item()
    diff = (stepped - full[:, 15:]).abs().max().item()
    print(f"cached vs cache-free max |dlogit| = {diff:.4f}; the oracle's own gap {gap_o:.4f}")
    assert diff <= 1.5 * gap_o + LOGIT_TOL
    agree_o = (stepped_o.argmax(-1) == full_o[:, 15:].argmax(-1)).float().mean().item()
    assert (stepped.argmax(-1) == full[:, 15:].argmax(-1)).float().mean().item() >= agree_o - 0.25
    # (the oracle's two attention forms only differ when there is a cache: a prefill into an empty cache is the same computation)
    floor_rel, floor_max, a, b = oracle_floor(rt, lambda r: gpt_ref.forward(r, seq_c, decode_ref.new_cache(r.cfg, 2, 24, torch.bfloat16)))
    assert_within_floor(full.cpu(), a, b, floor_rel, floor_max, "cache-free forward")


@pytest.mark.parametrize("cfg_kwargs,B", [(SMALL_MHA, 3), (SMALL_GQA, 70)])
def test_decode_from_an_empty_cache(cfg_kwargs, B):
    """One token per row per call from position 0: the first step's attention sees no cached key at all (every wave's run of
    keys is empty and the row attends to itself only), the next ones see 1, 2, ... keys."""
    say(f"decode from an empty cache {cfg_kwargs['n_embd']}/{cfg_kwargs['n_head']}q{cfg_kwargs['n_kv_head']}kv B={B}")
    rt, model = build_pair(cfg_kwargs, seed=11)
    from nanochat_amd.engine import KVCache
    cfg = rt.cfg
    g = torch.Generator().manual_seed(12)
    steps = 6
    ref = decode_ref.new_cache(cfg, B, steps, torch.bfloat16)
    rt_def = gpt_ref.Runtime(cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    ref_def = decode_ref.new_cache(cfg, B, steps, torch.bfloat16)
    dec = KVCache(B, cfg.n_kv_head, steps, 128, cfg.n_layer, DEV, torch.bfloat16)
    # whatever the cache memory holds must not matter before it is written
    dec.k_cache.fill_(float("nan"))
    dec.v_cache.fill_(float("nan"))
    S, Dd, G = [], [], []
    for s in range(steps):
        nxt = torch.randint(0, cfg.vocab_size, (B, 1), generator=g)
        S.append(gpt_ref.forward(rt, nxt, ref)[:, -1])
        Dd.append(gpt_ref.forward(rt_def, nxt, ref_def)[:, -1])
        G.append(model.forward_last(nxt.to(DEV), kv_cache=dec).cpu())
    S, Dd, G = torch.stack(S), torch.stack(Dd), torch.stack(G)
    assert torch.isfinite(G).all()
    assert_within_floor(G, S, Dd, rel_l2(Dd, S), (S - Dd).abs().max().item(), "decode from an empty cache")


@pytest.mark.parametrize("cfg_kwargs,B,P,steps", [(SMALL_GQA, 8, 40, 12), (SMALL_MHA, 5, 70, 10), (WIDE_GQA, 128, 90, 5),
                                                  (WIDE_MHA, 128, 3, 6)])
def test_small_models_batched_decode(cfg_kwargs, B, P, steps):
    say(f"small model {cfg_kwargs['n_embd']}/{cfg_kwargs['n_head']}q{cfg_kwargs['n_kv_head']}kv B={B}")
    rt, model = build_pair(cfg_kwargs, seed=3)
    from nanochat_amd.engine import KVCache
    cfg = rt.cfg
    g = torch.Generator().manual_seed(4)
    prompt = torch.randint(0, cfg.vocab_size, (1, P), generator=g)
    # the Engine's shape of work: prefill one row, replicate, decode B rows
    ref_pre = decode_ref.new_cache(cfg, 1, P, torch.bfloat16)
    want = gpt_ref.forward(rt, prompt, ref_pre)[:, -1].expand(B, -1)
    ref_dec = decode_ref.new_cache(cfg, B, P + steps, torch.bfloat16)
    ref_dec.prefill(ref_pre)
    pre = KVCache(1, cfg.n_kv_head, P, 128, cfg.n_layer, DEV, torch.bfloat16)
    got = model.forward_last(prompt.to(DEV), kv_cache=pre).expand(B, -1).cpu()
    dec = KVCache(B, cfg.n_kv_head, P + steps, 128, cfg.n_layer, DEV, torch.bfloat16)
    dec.prefill(pre)
    # positions that have not been written yet must never reach a result
    dec.k_cache[:, :, P:] = float("nan")
    dec.v_cache[:, :, P:] = float("nan")
    rt_def = gpt_ref.Runtime(cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    def_pre = decode_ref.new_cache(cfg, 1, P, torch.bfloat16)
    wdef = gpt_ref.forward(rt_def, prompt, def_pre)[:, -1].expand(B, -1)
    def_dec = decode_ref.new_cache(cfg, B, P + steps, torch.bfloat16)
    def_dec.prefill(def_pre)
    S, Dd, G = [want], [wdef], [got]
    for s in range(steps):
        nxt = torch.randint(0, cfg.vocab_size, (B, 1), generator=g)       # distinct tokens per row
        S.append(gpt_ref.forward(rt, nxt, ref_dec)[:, -1])
        Dd.append(gpt_ref.forward(rt_def, nxt, def_dec)[:, -1])
        G.append(model.forward_last(nxt.to(DEV), kv_cache=dec).cpu())
    S, Dd, G = torch.stack(S), torch.stack(Dd), torch.stack(G)
    assert_within_floor(G, S, Dd, rel_l2(Dd, S), (S - Dd).abs().max().item(), "prefill + batched decode")


LONG_GQA = dict(sequence_len=1024, vocab_size=1024, n_layer=4, n_head=4, n_kv_head=2, n_embd=512, window_pattern="SL")
LONG_MHA = dict(sequence_len=2048, vocab_size=2048, n_layer=3, n_head=3, n_kv_head=3, n_embd=384, window_pattern="SSL")


@pytest.mark.parametrize("cfg_kwargs,B,P,trained_like", [(LONG_GQA, 1, 200, True), (LONG_GQA, 2, 150, True), (LONG_MHA, 1, 700, True),
                                                         (LONG_MHA, 1, 1100, False), (LONG_GQA, 1, 520, False)])
def test_long_prefill_matches_oracle(cfg_kwargs, B, P, trained_like):
    """More than 128 rows in one forward: the tiled FP8 GEMMs (with the relu^2 epilogue), the convert pass, the stand-alone rotary
    kernel and the matrix-core attention, all positions' logits against the oracle; then two decode steps on that cache."""
    say(f"long prefill {cfg_kwargs['n_embd']}/{cfg_kwargs['n_head']}q{cfg_kwargs['n_kv_head']}kv B={B} P={P} trained_like={trained_like}")
    rt, model = build_pair(cfg_kwargs, seed=5, trained_like=trained_like)
    from nanochat_amd.engine import KVCache
    cfg = rt.cfg
    g = torch.Generator().manual_seed(6)
    prompt = torch.randint(0, cfg.vocab_size, (B, P), generator=g)
    steps = [torch.randint(0, cfg.vocab_size, (B, 1), generator=g) for _ in range(2)]

    def run(r):
        c = decode_ref.new_cache(cfg, B, P + 2, torch.bfloat16)
        outs = [gpt_ref.forward(r, prompt, c)]
        for nxt in steps:
            outs.append(gpt_ref.forward(r, nxt, c))
        return torch.cat(outs, dim=1)
    floor_rel, floor_max, want, want_def = oracle_floor(rt, run)
    cache = KVCache(B, cfg.n_kv_head, P + 2, 128, cfg.n_layer, DEV, torch.bfloat16)
    got = [model(prompt.to(DEV), kv_cache=cache).cpu()]
    for nxt in steps:
        got.append(model(nxt.to(DEV), kv_cache=cache).cpu())
    got = torch.cat(got, dim=1)
    assert got.shape == want.shape == (B, P + 2, cfg.vocab_size)
    if trained_like:
        assert_within_floor(got, want, want_def, floor_rel, floor_max, "long prefill logits")
    else:
        worst = min((got - want).abs().max().item(), (got - want_def).abs().max().item())
        assert worst <= LOGIT_TOL, worst
    assert cache.get_pos() == P + 2


def test_ragged_rows():
    """Per-row cache lengths (outside the reference's GPT.forward, inside FA3's signature): every row
    must equal the same row run alone."""
    say("ragged rows")
    rt, model = build_pair(SMALL_GQA, seed=5)
    from nanochat_amd.engine import KVCache
    cfg = rt.cfg
    g = torch.Generator().manual_seed(6)
    lens = [3, 17, 40, 9]
    B = len(lens)
    big = KVCache(B, cfg.n_kv_head, 64, 128, cfg.n_layer, DEV, torch.bfloat16)
    prevs = []
    prompts = [torch.randint(0, cfg.vocab_size, (1, n), generator=g) for n in lens]
    for b, pr in enumerate(prompts):
        one = KVCache(1, cfg.n_kv_head, 64, 128, cfg.n_layer, DEV, torch.bfloat16)
        model.forward_last(pr.to(DEV), kv_cache=one)
        big.k_cache[:, b] = one.k_cache[:, 0]
        big.v_cache[:, b] = one.v_cache[:, 0]
        prevs.append(one.prev_embedding)
    big.set_seqlens(lens)
    big.prev_embedding = torch.cat(prevs, dim=0)
    nxt = torch.randint(0, cfg.vocab_size, (B, 1), generator=g)
    got = model.forward_last(nxt.to(DEV), kv_cache=big).cpu()
    assert big.cache_seqlens.tolist() == [n + 1 for n in lens]
    # oracle, ragged mode
    rt2 = gpt_ref.Runtime(cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    ref_big = decode_ref.new_cache(cfg, B, 64, torch.bfloat16)
    rprev = []
    for b, pr in enumerate(prompts):
        one = decode_ref.new_cache(cfg, 1, 64, torch.bfloat16)
        gpt_ref.forward(rt, pr, one)
        ref_big.k_cache[:, b] = one.k_cache[:, 0]
        ref_big.v_cache[:, b] = one.v_cache[:, 0]
        rprev.append(one.prev_embedding)
    ref_big.cache_seqlens.copy_(torch.tensor(lens, dtype=torch.int32))
    ref_big.prev_embedding = torch.cat(rprev, dim=0)
    want = gpt_ref.forward(rt2, nxt, ref_big)[:, -1]
    # floor: the same rows through the SDPA oracle, one row at a time (the reference's only way to run them)
    singles = []
    for b, pr in enumerate(prompts):
        one = decode_ref.new_cache(cfg, 1, 64, torch.bfloat16)
        gpt_ref.forward(rt, pr, one)
        singles.append(gpt_ref.forward(rt, nxt[b:b + 1], one)[0, -1])
    singles = torch.stack(singles)
    # NB: row-at-a-time calls quantize each row with its own tensorwise scale, the batched call shares one
    # scale over the batch, so this floor also contains that (legitimate) difference.
    assert_within_floor(got, want, singles, max(rel_l2(singles, want), 0.03), (singles - want).abs().max().item(), "ragged rows")


def test_engine_generate_sampling_on_gpu(d4_pair):
    say("Engine.generate sampled, num_samples=8")
    rt, model = d4_pair
    from nanochat_amd.engine import Engine
    from test_engine_host import ByteTokenizer
    tok = ByteTokenizer()
    tok._special = {k: 32000 + i for i, k in enumerate(tok._special)}
    tok.get_bos_token_id = lambda: 32005
    engine = Engine(model, tok)
    prompt = [5, 99, 12345, 777, 31000]
    r1, m1 = engine.generate_batch(prompt, num_samples=8, max_tokens=12, temperature=1.0, top_k=50, seed=7)
    r2, _ = engine.generate_batch(prompt, num_samples=8, max_tokens=12, temperature=1.0, top_k=50, seed=7)
    r3, _ = engine.generate_batch(prompt, num_samples=8, max_tokens=12, temperature=1.0, top_k=50, seed=8)
    assert r1 == r2 and r1 != r3
    assert len(r1) == 8 and all(len(r) <= len(prompt) + 12 for r in r1)
    assert len({tuple(r) for r in r1}) > 1                       # rows sample independently
    g1, _ = engine.generate_batch(prompt, num_samples=4, max_tokens=8, temperature=0.0)
    assert all(r == g1[0] for r in g1)                           # greedy rows are identical


def test_engine_run_ahead_step_is_taken_back_when_a_token_is_forced(d4_pair):
    """Engine.generate enqueues the next forward on the sampled ids before the host has read them.  When the tool-use
    machine forces another token the step must be redone: a run whose rows get forced tokens at chosen steps has to
    match the same run through a model object without the fast path (the plain sample -> host -> forward loop)."""
    say("Engine.generate: forced tokens vs run-ahead forward")
    rt, model = d4_pair
    from nanochat_amd.engine import Engine
    from test_engine_host import ByteTokenizer
    tok = ByteTokenizer()
    tok._special = {k: 32000 + i for i, k in enumerate(tok._special)}
    tok.get_bos_token_id = lambda: 32005

    class Forcing(Engine):                  # forces a token for row 1 at steps 2 and 3, for every row at step 6
        def generate(self, *a, **k):
            self._calls = 0
            return super().generate(*a, **k)

        def _step_row(self, state, sampled, sp):
            step, row = divmod(self._calls, 4)
            self._calls += 1
            if (row == 1 and step in (2, 3)) or step == 6:
                state.forced_tokens.append((sampled + 17 + row) % 30000)
            return super()._step_row(state, sampled, sp)

    class PlainModel:                       # same model, no forward_last: the engine takes the plain loop
        def __init__(self, m):
            self.config, self._m = m.config, m

        def get_device(self):
            return self._m.get_device()

        def forward(self, ids, kv_cache=None):
            return self._m.forward(ids, kv_cache=kv_cache)

    prompt = [5, 99, 12345, 777, 31000, 42]
    for temperature, top_k in ((0.0, None), (0.9, 40)):
        runs = []
        for m in (model, PlainModel(model)):
            cols = list(Forcing(m, tok).generate(prompt, num_samples=4, max_tokens=10, temperature=temperature, top_k=top_k, seed=3))
            runs.append(cols)
        assert runs[0] == runs[1]
        assert any(0 in masks for _, masks in runs[0])          # forced tokens did occur
        assert len(runs[0]) == 10


def test_model_refuses_what_it_does_not_implement(d4_pair):
    rt, model = d4_pair
    from nanochat_amd.gpt import GPT, GPTConfig
    idx = torch.zeros(1, 4, dtype=torch.long, device=DEV)
    with pytest.raises(NotImplementedError):
        model(idx, targets=idx)
    with pytest.raises(RuntimeError):
        model(idx.cpu())
    plain = GPT(GPTConfig(**SMALL_MHA)).to(DEV)
    with pytest.raises(RuntimeError):
        plain(idx)                                               # not converted to FP8
    from nanochat_amd.engine import KVCache
    tiny = KVCache(1, 2, 3, 128, 4, DEV, torch.bfloat16)
    with pytest.raises(AssertionError):
        model(idx, kv_cache=tiny)                                # 4 tokens into a 3-slot cache


# ------------------------------------------------------------------------------------------------
# Full size (d26, 64 rows, context to 2048): no oracle can be run at this size in test time, so the checks are
# properties that hold whatever the size.
def test_full_size_d26_batch64_properties():
    say("d26 batch 64 full-size properties")
    from nanochat_amd.engine import KVCache
    from nanochat_amd.synthetic import config_for_depth, random_init_model
    cfg = config_for_depth(26)
    model = random_init_model(cfg, DEV, seed=2)
    B, P = 64, 1792
    g = torch.Generator().manual_seed(7)
    prompt = torch.randint(0, cfg.vocab_size, (1, P), generator=g).to(DEV)
    pre = KVCache(1, cfg.n_kv_head, P, 128, cfg.n_layer, DEV, torch.bfloat16)
    first = model.forward_last(prompt, kv_cache=pre)
    assert first.shape == (1, cfg.vocab_size) and torch.isfinite(first).all()
    dec = KVCache(B, cfg.n_kv_head, 2048, 128, cfg.n_layer, DEV, torch.bfloat16)
    dec.prefill(pre)
    # (1) replicated rows fed the same tokens compute the same thing: logits identical across the 64 rows, bit for bit
    tok = first.argmax(-1, keepdim=True).expand(B, 1).contiguous()
    steps = []
    for _ in range(3):
        logits = model.forward_last(tok, kv_cache=dec)
        assert logits.shape == (B, cfg.vocab_size) and torch.isfinite(logits).all()
        assert torch.equal(logits, logits[:1].expand(B, -1)), "rows of one replicated prompt diverged"
        steps.append(logits[0].clone())
        tok = logits.argmax(-1, keepdim=True)
    assert dec.get_pos() == P + 3 and dec.cache_seqlens.tolist() == [P + 3] * B
    # (2) cached decode equals one forward over the longer sequence: position P of a (P+1)-token prefill sees the same
    # keys and values as the first decode step (different kernels, same mathematics; fp8 and bf16 rounding apart)
    longer = torch.cat([prompt, first.argmax(-1, keepdim=True)], dim=1)
    pre2 = KVCache(1, cfg.n_kv_head, P + 1, 128, cfg.n_layer, DEV, torch.bfloat16)
    full = model.forward_last(longer, kv_cache=pre2)[0]
    rel = rel_l2(steps[0], full)
    print(f"d26: decode step vs (P+1)-token prefill rel-L2 {rel:.4f}, argmax {steps[0].argmax().item()} / {full.argmax().item()}")
    assert rel < 0.1
    # the appended cache rows agree with the prefill's rows for the same position up to fp8 noise (the tensorwise scale of
    # a 64-row decode batch is not that of a 1793-row prefill, so not bit for bit)
    for layer in (0, cfg.n_layer - 1):
        assert rel_l2(dec.k_cache[layer, 0, P], pre2.k_cache[layer, 0, P]) < 0.1
        assert rel_l2(dec.v_cache[layer, 0, P], pre2.v_cache[layer, 0, P]) < 0.1
    # (3) a row with a different token diverges from the others, and does not disturb them: rows are independent
    # apart from the shared tensorwise scales
    tok2 = tok.clone()
    tok2[5, 0] = (tok2[5, 0] + 1234) % cfg.vocab_size
    snap = dec.cache_seqlens.clone()
    l_mixed = model.forward_last(tok2, kv_cache=dec)
    assert not torch.equal(l_mixed[5], l_mixed[0])
    assert torch.equal(l_mixed[0], l_mixed[63]) and torch.equal(snap + 1, dec.cache_seqlens)


@pytest.mark.parametrize("K,N", [(1664, 4992), (1664, 1664), (1664, 6656), (6656, 1664)])
def test_full_size_float8linear_shapes_against_fp32_matmul(K, N):
    """The isolated Float8Linear shapes at M = 8192, forward and both backward GEMMs, against torch's fp32 matmul of the
    same fp8 payloads on the GPU (the CPU oracle covers smaller sizes; payloads are checked bit for bit elsewhere)."""
    say(f"full-size Float8Linear M=8192 K={K} N={N}")
    from nanochat_amd import ops
    M = 8192
    g = torch.Generator(device=DEV).manual_seed(K + N)
    a = torch.randn(M, K, device=DEV, generator=g)
    a = torch.where(torch.rand(M, K, device=DEV, generator=g) < 0.001, a * 20, a).bfloat16()
    w = ((torch.rand(N, K, device=DEV, generator=g) * 2 - 1) * (3.0 / K) ** 0.5).bfloat16()
    go = (torch.randn(M, N, device=DEV, generator=g) * 1e-3).bfloat16()
    a8, ia, _ = ops.fp8_quantize(a)
    w8, iw, _ = ops.fp8_quantize(w)
    go8, igo, _ = ops.fp8_quantize(go, fp8_dtype=torch.float8_e5m2)
    torch.backends.cuda.matmul.allow_tf32 = False
    af, wf, gf = a8.float(), w8.float(), go8.float()
    out = ops.fp8_gemm(a8, w8, ia, iw.reshape(1))
    assert rel_l2(out, (af @ wf.t()) * ia * iw) <= 3e-3
    gi = ops.fp8_gemm_grad(go8, ops.fp8_transpose(w8), igo, iw)
    assert rel_l2(gi, (gf @ wf) * igo * iw) <= 3e-3
    gw = ops.fp8_gemm_grad(ops.fp8_transpose(go8), ops.fp8_transpose(a8), igo, ia)
    assert rel_l2(gw, (gf.t() @ af) * igo * ia) <= 3e-3
    # linearity in the scales: doubling an inverse scale doubles the result exactly (power of two)
    out2 = ops.fp8_gemm(a8, w8, ia * 2, iw.reshape(1))
    assert torch.equal(out2.float(), out.float() * 2)


def test_full_size_d32_gqa_batch128_ragged_rows():
    """d32 with 16 query / 4 kv heads, 128 rows of lengths in [64, 2048): rows that hold the same history and get the same
    token give the same logits wherever they sit in the batch, a row's result does not depend on what the other rows hold
    beyond the shared tensorwise scales, and the whole batch agrees with running a few rows in a batch of their own."""
    say("d32 GQA batch 128 ragged full-size properties")
    from nanochat_amd.engine import KVCache
    from nanochat_amd.synthetic import config_for_depth, random_init_model
    cfg = config_for_depth(32, n_kv_head=4)
    assert (cfg.n_embd, cfg.n_head, cfg.n_kv_head) == (2048, 16, 4)
    model = random_init_model(cfg, DEV, seed=3)
    B, Tmax = 128, 2048
    g = torch.Generator().manual_seed(8)
    lens = torch.randint(64, 2048, (B,), generator=g).tolist()
    lens[1], lens[77], lens[126] = lens[0], lens[0], lens[5]          # duplicates of rows 0 and 5
    gd = torch.Generator(device=DEV).manual_seed(9)
    cache = KVCache(B, cfg.n_kv_head, Tmax, 128, cfg.n_layer, DEV, torch.bfloat16)
    cache.k_cache.normal_(0.0, 1.0, generator=gd)
    cache.v_cache.normal_(0.0, 1.0, generator=gd)
    for dup, src in ((1, 0), (77, 0), (126, 5)):
        cache.k_cache[:, dup] = cache.k_cache[:, src]
        cache.v_cache[:, dup] = cache.v_cache[:, src]
    prev = torch.randn(B, 1, cfg.n_embd, device=DEV, generator=gd).bfloat16()
    prev[1], prev[77], prev[126] = prev[0], prev[0], prev[5]
    cache.set_seqlens(lens)
    cache.prev_embedding = prev.clone()
    tok = torch.randint(0, cfg.vocab_size, (B, 1), generator=g).to(DEV)
    tok[1], tok[77], tok[126] = tok[0], tok[0], tok[5]
    k_before = cache.k_cache[:, :, :64].clone()
    logits = model.forward_last(tok, kv_cache=cache)
    assert logits.shape == (B, cfg.vocab_size) and torch.isfinite(logits).all()
    assert cache.cache_seqlens.tolist() == [n + 1 for n in lens]
    assert torch.equal(logits[0], logits[1]) and torch.equal(logits[0], logits[77]) and torch.equal(logits[5], logits[126])
    assert not torch.equal(logits[0], logits[5])
    assert torch.equal(cache.k_cache[:, :, :64], k_before)                     # the append touched position len only
    # the same rows in a batch of four: same mathematics, other tensorwise scales
    pick = [0, 5, 40, 127]
    small = KVCache(len(pick), cfg.n_kv_head, Tmax, 128, cfg.n_layer, DEV, torch.bfloat16)
    for i, b in enumerate(pick):
        small.k_cache[:, i] = cache.k_cache[:, b]
        small.v_cache[:, i] = cache.v_cache[:, b]
    small.set_seqlens([lens[b] for b in pick])
    small.prev_embedding = prev[pick].clone()
    l4 = model.forward_last(tok[pick], kv_cache=small)
    rel = rel_l2(l4, logits[pick])
    print(f"d32 GQA: rows in a batch of 4 vs in the batch of 128: rel-L2 {rel:.4f}")
    assert rel < 0.1


@pytest.mark.parametrize("B", [1, 3, 40])
def test_positions_advanced_inside_the_step_or_by_the_caller(B):
    """A one-token forward may advance cache_seqlens inside its last row kernel (nc_cache_desc.advance) instead of leaving it to the
    caller: same logits, same positions, same cache, for the fused small-batch step (1 row), the split linears (3) and the unsplit
    c_fc (40 rows)."""
    say(f"positions advanced inside the step, {B} row(s)")
    from nanochat_amd.engine import KVCache

    class CallerAdvances(KVCache):
        """A cache without note_advanced(): GPT.forward then leaves advance = 0 and calls advance() itself."""
        def __getattribute__(self, name):
            if name == "note_advanced":
                raise AttributeError(name)
            return super().__getattribute__(name)

    cfg_kwargs = dict(sequence_len=64, vocab_size=1024, n_layer=3, n_head=4, n_kv_head=2, n_embd=512, window_pattern="SL")
    _, model = build_pair(cfg_kwargs, seed=43)
    g = torch.Generator().manual_seed(44)
    P, steps = 7, 4
    prompt = torch.randint(0, 1024, (B, P), generator=g).to(DEV)
    toks = [torch.randint(0, 1024, (B, 1), generator=g).to(DEV) for _ in range(steps)]
    caches = [cls(B, 2, P + steps + 1, 128, 3, DEV, torch.bfloat16) for cls in (KVCache, CallerAdvances)]
    assert hasattr(caches[0], "note_advanced") and not hasattr(caches[1], "note_advanced")
    outs = []
    for c in caches:
        got = [model.forward_last(prompt, kv_cache=c).clone()]
        for t in toks:
            got.append(model.forward_last(t, kv_cache=c).clone())
            assert c.get_pos() == int(c.cache_seqlens[0])                 # the host mirror follows either way
        outs.append(got)
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    assert torch.equal(caches[0].cache_seqlens, caches[1].cache_seqlens)
    assert int(caches[0].cache_seqlens[B - 1]) == P + steps
    assert torch.equal(caches[0].k_cache, caches[1].k_cache) and torch.equal(caches[0].v_cache, caches[1].v_cache)


def test_weight_changes_are_noticed_by_the_next_forward():
    """The quantized copies of the FP8 weights are cached between calls; every way of changing a weight that the module API offers
    must refresh them: an in-place update, load_state_dict (copying and assigning), a cast of a child module, and the explicit call
    for a parameter assigned by hand."""
    say("weight plan refresh")
    from nanochat_amd.engine import KVCache
    cfg_kwargs = dict(sequence_len=64, vocab_size=512, n_layer=2, n_head=2, n_kv_head=2, n_embd=256, window_pattern="L")
    _, model = build_pair(cfg_kwargs, seed=31)
    ids = torch.arange(12, device=DEV).reshape(1, 12) * 5 % 512

    def logits():
        return model.forward_last(ids, kv_cache=KVCache(1, 2, 16, 128, 2, DEV, torch.bfloat16)).clone()
    base = logits()
    assert torch.equal(base, logits())                                   # cached plan, same answer
    w = model.transformer.h[1].mlp.c_proj.weight
    with torch.no_grad():
        w.mul_(1.5)                                                      # in place: version counter
    changed = logits()
    assert not torch.equal(changed, base)
    state = {k: v.clone() for k, v in model.state_dict().items()}
    with torch.no_grad():
        w.mul_(1.0 / 1.5)
    restored = logits()
    assert not torch.equal(restored, changed)
    model.load_state_dict(state)                                         # copy into the existing tensors
    assert torch.equal(logits(), changed)
    with torch.no_grad():
        w.mul_(1.0 / 1.5)
    model.load_state_dict(state, assign=True)                            # new parameter objects
    assert torch.equal(logits(), changed)
    model.lm_head.weight = torch.nn.Parameter(model.lm_head.weight.detach() * 2.0)      # a new parameter object, assigned by hand
    doubled = logits()
    assert not torch.equal(doubled, changed), "a replaced parameter object went unnoticed: the forward used stale e4m3 weights"
    blk = model.transformer.h[0].mlp.c_fc
    blk.weight = torch.nn.Parameter(blk.weight.detach() * 0.5)
    halved = logits()
    assert not torch.equal(halved, doubled)
    blk.weight = torch.nn.Parameter(blk.weight.detach() * 2.0)
    assert torch.equal(logits(), doubled)
    model.value_embeds.to(torch.float32)                                 # a child cast: same parameter objects, new storage
    model.value_embeds.to(torch.bfloat16)
    assert torch.equal(logits(), doubled)


def test_engine_generate_reading_the_shared_prompt_once():
    """Engine.generate(share_prompt_reads=True): every row's cache starts with a copy of the one prompt, and the full-context layers
    read that copy once for all rows.  On the repository init (attention contributes nothing to the logits there) the token stream is
    that of the plain loop; on a trained-like model the logits of a decode step agree with the per-row path to the distance at which
    the oracle's own two attention forms agree, and with the oracle."""
    say("shared prompt: Engine.generate with share_prompt_reads")
    from nanochat_amd.engine import Engine, KVCache
    from test_engine_host import ByteTokenizer

    class Tok(ByteTokenizer):
        def __init__(self):
            self._special = {"<|python_start|>": 2040, "<|python_end|>": 2041, "<|output_start|>": 2042,
                             "<|output_end|>": 2043, "<|assistant_end|>": 2044, "<|bos|>": 2045}

        def get_bos_token_id(self):
            return 2045
    # 64 rows x 8 kv heads: the per-row kernel runs unsplit, which the shared form needs; three of four layers are full-context
    cfg = dict(sequence_len=2048, vocab_size=2048, n_layer=4, n_head=8, n_kv_head=8, n_embd=1024, window_pattern="LLSL")
    g = torch.Generator().manual_seed(5)
    prompt = torch.randint(0, 2000, (900,), generator=g).tolist()
    rt, model = build_pair(cfg, seed=31, trained_like=False)
    runs = []
    for share in (False, True):
        cols = [c for c, _ in Engine(model, Tok()).generate(prompt, num_samples=64, max_tokens=24, temperature=1.0, top_k=50, seed=7,
                                                           share_prompt_reads=share)]
        runs.append(cols)
    assert runs[0] == runs[1] and len(runs[0]) == 24
    # trained-like weights: one decode step, both ways, and the oracle on a few rows
    rt, model = build_pair(cfg, seed=32, trained_like=True)
    B, P = 64, 900
    ids = torch.tensor([prompt])
    pre = KVCache(1, 8, P, 128, 4, DEV, torch.bfloat16)
    model.forward_last(ids.to(DEV), kv_cache=pre)
    nxt = torch.randint(0, 2000, (B, 1), generator=g)
    outs = {}
    for share in (False, True):
        dec = KVCache(B, 8, P + 8, 128, 4, DEV, torch.bfloat16, prefill_from=pre, share_prompt_reads=share)
        assert dec.shared_prefix_len == P
        a = model.forward_last(nxt.to(DEV), kv_cache=dec).cpu()
        b = model.forward_last(nxt.roll(1, 0).to(DEV), kv_cache=dec).cpu()      # a second step: the rows' own tails now hold two tokens
        outs[share] = torch.stack([a, b])
    rows = [0, 13, 63]
    ref = decode_ref.new_cache(rt.cfg, 1, P + 8, torch.bfloat16)
    gpt_ref.forward(rt, ids, ref)
    big = decode_ref.new_cache(rt.cfg, len(rows), P + 8, torch.bfloat16)
    big.prefill(ref)
    rt_def = gpt_ref.Runtime(rt.cfg, rt.p, compute_dtype=torch.bfloat16, fp8=True, uniform_sdpa=False)
    big_def = decode_ref.new_cache(rt.cfg, len(rows), P + 8, torch.bfloat16)
    big_def.prefill(ref)
    want = torch.stack([gpt_ref.forward(rt, nxt[rows], big)[:, -1], gpt_ref.forward(rt, nxt.roll(1, 0)[rows], big)[:, -1]])
    want_def = torch.stack([gpt_ref.forward(rt_def, nxt[rows], big_def)[:, -1], gpt_ref.forward(rt_def, nxt.roll(1, 0)[rows], big_def)[:, -1]])
    floor_rel, floor_max = rel_l2(want_def, want), (want - want_def).abs().max().item()
    # (the oracle quantizes with the amax of 3 rows, the GPU with that of 64: the floor criterion covers both differences)
    print(f"shared prompt vs per-row path: rel_l2 {rel_l2(outs[True], outs[False]):.4f} max {(outs[True] - outs[False]).abs().max().item():.4f}")
    assert_within_floor(outs[True][:, rows], want, want_def, max(floor_rel, rel_l2(outs[False][:, rows], want)), floor_max, "shared-prompt decode")
    assert rel_l2(outs[True], outs[False]) <= 1.5 * max(floor_rel, rel_l2(outs[False][:, rows], want)) + 1e-3
    # (the two paths sum in different orders and the shared part's weights pass through bf16: equal bits would mean that the
    # shared form had not run at all)
    assert not torch.equal(outs[True], outs[False]), "the shared-prompt path was meant to run for this shape"


@pytest.mark.parametrize("B", [4, 1])
def test_decode_step_captured_in_a_graph_replays_like_the_eager_step(B):
    """The decode forward makes no allocation of its own, clears its counters with a kernel and reads positions from device memory,
    so a caller may capture it in a HIP graph.  Replayed several times, with eager work and synchronisations in between, every replay
    must give the logits and the cache of the eager step bit for bit."""
    say(f"decode step under graph capture, {B} row(s)")
    from nanochat_amd.engine import KVCache
    cfg_kwargs = dict(sequence_len=64, vocab_size=1024, n_layer=3, n_head=4, n_kv_head=2, n_embd=512, window_pattern="SL")
    _, model = build_pair(cfg_kwargs, seed=41)
    P, steps = 9, 5
    g = torch.Generator().manual_seed(42)
    prompt = torch.randint(0, 1024, (B, P), generator=g).to(DEV)
    toks = [torch.randint(0, 1024, (B, 1), generator=g).to(DEV) for _ in range(steps)]

    def fresh():
        c = KVCache(B, 2, P + steps + 1, 128, 3, DEV, torch.bfloat16)
        model.forward_last(prompt, kv_cache=c)
        return c
    eager, graphed, scratch = fresh(), fresh(), fresh()
    static_idx = torch.zeros(B, 1, dtype=torch.long, device=DEV)
    static_prev = graphed.prev_embedding.clone()          # the smear state lives in one buffer that the graph updates itself
    graphed.prev_embedding = static_prev
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                           # warm-up of the step's workspace outside the capture
        model.forward_last(toks[0], kv_cache=scratch)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_logits = model.forward_last(static_idx, kv_cache=graphed)
        static_prev.copy_(graphed.prev_embedding)
    graphed.prev_embedding = static_prev
    # the capture advanced the host mirror of the position and, being a capture, nothing on the device
    graphed._pos0 -= 1
    graphed._pos_max -= 1
    assert int(graphed.cache_seqlens[0]) == P
    for step, tok in enumerate(toks):
        want = model.forward_last(tok, kv_cache=eager).clone()     # the program's own eager work between the replays
        torch.cuda.synchronize()
        static_idx.copy_(tok)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static_logits, want), f"replay {step}: max |diff| {(static_logits - want).abs().max().item()}"
        assert torch.equal(graphed.cache_seqlens, eager.cache_seqlens)
    assert torch.equal(graphed.k_cache[:, :, :P + steps], eager.k_cache[:, :, :P + steps])
    assert torch.equal(graphed.v_cache[:, :, :P + steps], eager.v_cache[:, :, :P + steps])

