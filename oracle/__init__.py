"""CPU oracle for the FP8 + KV-cache decode path.

TEST INFRASTRUCTURE ONLY.  Nothing in ``nanochat_amd`` may import this package:
it exists so that tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg
of ``bench.py`` can check the HIP path against an independent restatement of the
reference semantics, written with plain torch CPU ops (and one small C file for
the e4m3 encoder).

Modules
-------
fp8_ref        tensorwise e4m3 quantize and the fp8-emulated matmul
               (nanochat/fp8.py:81-107, 132-154, 195-266)
e4m3.c         bit-level C restatement of the same quantizer (no torch)
attention_ref  KV-cache attention with sliding window and GQA
               (nanochat/flash_attention.py:77-110, 139-185)
gpt_ref        functional GPT forward over a reference-named state dict
               (nanochat/gpt.py:28-65, 84-153, 204-314, 459-524)
decode_ref     KV cache container, sampler and a minimal generate loop
               (nanochat/engine.py:82-156, 175-275)

Pinning status (what each function is checked against, besides the HIP path):
  to_fp8 ............ torch's own ``.to(float8_e4m3fn)`` over all 65536 bf16 bit
                      patterns, e4m3.c, closed-form special cases, and golden
                      vectors written by the reference's ``_to_fp8``.
  scaled_mm ......... ``torch._scaled_mm`` on CPU (library routine), exact
                      power-of-two cases, brute force at K=16.
  rms_norm, rotary .. ``F.rms_norm`` / closed forms and invariants.
  attention ......... brute-force softmax, ``F.scaled_dot_product_attention``.
  gpt forward ....... golden logits/ids written by the reference's own GPT
                      (tests/golden), plus cached-decode == full-forward.
  sampler ........... ``torch.multinomial`` identity, argmax first-index rule.
"""
