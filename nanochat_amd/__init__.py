"""nanochat_amd: the FP8 + KV-cache decode hot path of nanochat, built for MI355X (gfx950).

Python keeps the reference's API (Float8Linear, GPT.forward(idx, kv_cache=...), KVCache,
Engine.generate, flash_attn.flash_attn_with_kvcache); the work is done by hand-written HIP kernels
in libnanochat_amd.so, reached through the C ABI declared in include/nanochat_amd.h.
"""
from .common import COMPUTE_DTYPE  # noqa: F401
