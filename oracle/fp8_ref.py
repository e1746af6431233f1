"""Oracle: tensorwise e4m3 quantize + fp8-emulated matmul (torch CPU).

Test infrastructure only; never imported by the product package.

Follows nanochat/fp8.py:81-107 (``_to_fp8``), :132-154 (``_Float8Matmul.forward``)
and :202-213 (``Float8Linear.forward``).
"""
import torch

E4M3_MAX = 448.0          # torch.finfo(torch.float8_e4m3fn).max
AMAX_FLOOR = 1e-12        # nanochat/fp8.py:78


def to_fp8(x: torch.Tensor):
    """(payload e4m3fn, inv_scale fp32 0-dim, scale fp32 0-dim) for one tensor.

    nanochat/fp8.py:91-106: amax in fp32, 448/amax in fp64 rounded to fp32,
    x*scale in fp32, saturate to +-448, round-to-nearest-even cast.
    """
    amax = x.float().abs().max()
    scale = (E4M3_MAX / amax.double().clamp(min=AMAX_FLOOR)).float()
    payload = (x.float() * scale).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn)
    return payload, scale.reciprocal(), scale


def scaled_mm_emulated(a8, w8, inv_a, inv_w, out_dtype=torch.bfloat16):
    """out[M,N] = out_dtype((a8 @ w8^T in fp32) * inv_a * inv_w), a8 [M,K], w8 [N,K]."""
    acc = a8.float() @ w8.float().t()
    return (acc * inv_a * inv_w).to(out_dtype)


def scaled_mm_library(a8, w8, inv_a, inv_w, out_dtype=torch.bfloat16):
    """The call the reference makes (nanochat/fp8.py:143-153), on CPU."""
    return torch._scaled_mm(a8, w8.t(), scale_a=inv_a, scale_b=inv_w,
                            out_dtype=out_dtype, use_fast_accum=True)


class WeightCache:
    """Memoises quantized weights by (data_ptr, version).

    The reference re-quantizes the weight on every forward (fp8.py:136); for a
    frozen weight the result is identical, so tests may cache it to save time.
    """

    def __init__(self):
        self._store = {}

    def get(self, w):
        key = (w.data_ptr(), w._version, tuple(w.shape), w.dtype)
        hit = self._store.get(key)
        if hit is None:
            p, inv, _ = to_fp8(w)
            hit = (p, inv)
            self._store[key] = hit
        return hit


def float8_linear(x, weight, compute_dtype=torch.bfloat16, wcache=None, library=False):
    """Float8Linear.forward without bias (nanochat/fp8.py:202-213)."""
    x = x.to(compute_dtype)
    shape = x.shape
    x2 = x.reshape(-1, shape[-1])
    a8, inv_a, _ = to_fp8(x2)
    if wcache is not None:
        w8, inv_w = wcache.get(weight)
    else:
        w8, inv_w, _ = to_fp8(weight)
    mm = scaled_mm_library if library else scaled_mm_emulated
    out = mm(a8, w8, inv_a, inv_w, out_dtype=x2.dtype)
    return out.reshape(*shape[:-1], out.shape[-1])


def fp8_module_filter(in_features, out_features):
    """Which linears get converted (scripts/base_train.py:178-185)."""
    return (in_features % 16 == 0 and out_features % 16 == 0
            and min(in_features, out_features) >= 128)
