"""Oracle: tensorwise fp8 quantize + fp8-emulated matmul, forward and backward (torch CPU).

Test infrastructure only; never imported by the product package.

Follows nanochat/fp8.py:81-107 (``_to_fp8``), :132-154 (``_Float8Matmul.forward``), :156-192
(``_Float8Matmul.backward``) and :202-213 (``Float8Linear.forward``).
"""
import torch

E4M3_MAX = 448.0          # torch.finfo(torch.float8_e4m3fn).max
E5M2_MAX = 57344.0        # torch.finfo(torch.float8_e5m2).max
AMAX_FLOOR = 1e-12        # nanochat/fp8.py:78


def to_fp8(x: torch.Tensor, fp8_dtype=torch.float8_e4m3fn):
    """(payload, inv_scale fp32 0-dim, scale fp32 0-dim) for one tensor.

    nanochat/fp8.py:91-106: amax in fp32, fp8_max/amax in fp64 rounded to fp32,
    x*scale in fp32, saturate to +-fp8_max, round-to-nearest-even cast.  e4m3fn for
    activations and weights, e5m2 for gradients (nanochat/fp8.py:165).
    """
    fmax = E4M3_MAX if fp8_dtype == torch.float8_e4m3fn else E5M2_MAX
    amax = x.float().abs().max()
    scale = (fmax / amax.double().clamp(min=AMAX_FLOOR)).float()
    payload = (x.float() * scale).clamp(-fmax, fmax).to(fp8_dtype)
    return payload, scale.reciprocal(), scale


def e5m2_encode_bits(y: torch.Tensor) -> torch.Tensor:
    """Round-to-nearest-even fp32 -> OCP e5m2 bytes by integer arithmetic, for |y| <= 57344 (the
    values _to_fp8 produces after its clamp).  A second, independent statement of the cast at
    nanochat/fp8.py:103 for the gradient format: e5m2 is the top byte of fp16, so the fp32 value
    is rounded to 2 mantissa bits above 2^-14 and to multiples of 2^-16 below."""
    bits = y.float().contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    sign = (bits >> 24) & 0x80
    mag = bits & 0x7FFFFFFF
    exp = (mag >> 23) - 127
    out = torch.zeros_like(mag)
    normal = exp >= -14
    # normal range: keep 2 mantissa bits, round to nearest even on the 21 dropped bits
    m = mag[normal]
    lsb = (m >> 21) & 1
    r = (m + 0xFFFFF + lsb) >> 21                 # (exponent+127) << 2 | mantissa, after rounding
    out[normal] = r - ((127 - 15) << 2)
    # subnormal range: value / 2^-16 rounded to nearest even integer 0..4
    sub = ~normal
    v = y.float().abs()[sub].double() * 65536.0
    q = torch.round(v)                             # torch.round is half-to-even
    out[sub] = q.to(torch.int64)
    return (out | sign).to(torch.uint8)


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


def float8_matmul_backward(grad_output, in_fp8, in_inv, w_fp8, w_inv):
    """_Float8Matmul.backward (nanochat/fp8.py:156-192) with fp8-emulated fp32 matmuls.

    grad_output [B,N] in the compute dtype; in_fp8 [B,K], w_fp8 [N,K] are the e4m3 payloads the forward saved.
    Returns (grad_input [B,K], grad_weight [N,K]) in grad_output's dtype, and the e5m2 payload and inverse scale
    of the gradient.  The reference's _to_col_major / .t().contiguous() only change the memory layout."""
    go_fp8, go_inv, _ = to_fp8(grad_output, torch.float8_e5m2)
    g = go_fp8.float()
    grad_input = ((g @ w_fp8.float()) * go_inv * w_inv).to(grad_output.dtype)
    grad_weight = ((g.t() @ in_fp8.float()) * go_inv * in_inv).to(grad_output.dtype)
    return grad_input, grad_weight, go_fp8, go_inv


def float8_matmul_backward_library(grad_output, in_fp8, in_inv, w_fp8, w_inv):
    """The three calls the reference makes (nanochat/fp8.py:165-190), on CPU."""
    go_fp8, go_inv, _ = to_fp8(grad_output, torch.float8_e5m2)
    w_col = w_fp8.t().contiguous().t()
    grad_input = torch._scaled_mm(go_fp8, w_col, scale_a=go_inv, scale_b=w_inv, out_dtype=grad_output.dtype, use_fast_accum=False)
    go_t = go_fp8.t().contiguous()
    in_col = in_fp8.t().contiguous().t()
    grad_weight = torch._scaled_mm(go_t, in_col, scale_a=go_inv, scale_b=in_inv, out_dtype=grad_output.dtype, use_fast_accum=False)
    return grad_input, grad_weight
