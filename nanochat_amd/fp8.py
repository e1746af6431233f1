"""Float8Linear on MI355X: tensorwise fp8 quantization + FP8 MFMA GEMMs.

Same public surface as nanochat/fp8.py (Float8Linear :195-227, Float8LinearConfig :230-240,
convert_to_float8_training :243-266).  Differences that do not change results:
  * the weight is quantized once and kept (payload + inverse scale) until the parameter's storage or
    version counter changes; the reference re-quantizes it on every call (fp8.py:136), which for an
    unchanged weight produces the same bytes;
  * without autograd (inference) no tensors are saved and the call is three launches; with autograd the
    three GEMMs of _Float8Matmul (fp8.py:123-192) run: e4m3 x e4m3 forward, e5m2 x e4m3 for both gradients,
    their transposed operands written by the quantization passes themselves instead of by separate copies.
"""
import torch
import torch.nn as nn

from . import ops
from .common import COMPUTE_DTYPE


class _Float8Matmul(torch.autograd.Function):
    """input_2d [B,K] @ weight[N,K]^T with the reference's three FP8 GEMMs (nanochat/fp8.py:123-192).

    The backward GEMMs want the summed index contiguous in both operands, which the reference gets from _to_col_major /
    .t().contiguous() copies (fp8.py:110-118,169,181-182).  Here every quantization that feeds the backward writes its payload
    both ways from one read of the bf16 tensor: the forward saves the input already transposed (when the weight needs a gradient),
    the output gradient is quantized to e5m2 once into [B,N] and [N,B], and the transposed weight payload is kept with the module's
    cached e4m3 weight.  Same payload bits and scales as the separate quantize + transpose passes."""

    @staticmethod
    def forward(ctx, input_2d, weight, module):
        rows, _ = input_2d.shape
        both_ways = weight.requires_grad and rows % 16 == 0
        if both_ways:
            a8, a8_t, inv_a, _ = ops.fp8_quantize_transposed(input_2d)
        else:
            a8, inv_a, _ = ops.fp8_quantize(input_2d)
            a8_t = None
        w8, inv_w = module._weight_fp8()
        ctx.module = module
        ctx.input_saved_transposed = a8_t is not None
        ctx.save_for_backward(a8_t if a8_t is not None else a8, inv_a, w8, inv_w)
        return ops.fp8_gemm(a8, w8, inv_a, inv_w)

    @staticmethod
    def backward(ctx, grad_output):
        a_saved, inv_a, w8, inv_w = ctx.saved_tensors
        if grad_output.dtype != torch.bfloat16:
            raise ValueError("Float8Linear: the GPU path computes in bf16")
        grad_output = grad_output.contiguous()
        need_in, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        # gradients in e5m2 (wider range), saved operands in e4m3 (fp8.py:163-165)
        go8_t = None
        if need_w and grad_output.shape[0] % 16 == 0:
            go8, go8_t, inv_go, _ = ops.fp8_quantize_transposed(grad_output, fp8_dtype=torch.float8_e5m2)
        else:
            go8, inv_go, _ = ops.fp8_quantize(grad_output, fp8_dtype=torch.float8_e5m2)
        grad_input = grad_weight = None
        if need_in:
            # grad_input [B,K] = grad_output [B,N] @ weight [N,K]: the summed index N must be contiguous in both (fp8.py:166-177)
            grad_input = ops.fp8_gemm_grad(go8, ctx.module._weight_fp8_transposed(w8), inv_go, inv_w)
        if need_w:
            # grad_weight [N,K] = grad_output^T [N,B] @ input [B,K]: B contiguous in both (fp8.py:179-190)
            if go8_t is None:
                go8_t = ops.fp8_transpose(go8)
            a8_t = a_saved if ctx.input_saved_transposed else ops.fp8_transpose(a_saved)
            grad_weight = ops.fp8_gemm_grad(go8_t, a8_t, inv_go, inv_a)
        return grad_input, grad_weight, None


class Float8Linear(nn.Linear):
    """nn.Linear whose matmul runs in FP8 on the GPU (fp8.py:195-213)."""

    def _weight_fp8(self):
        w = self.weight
        key = (w.data_ptr(), w._version, w.dtype, tuple(w.shape))
        cached = getattr(self, "_fp8_cache", None)
        if cached is None or cached[0] != key:
            with torch.no_grad():
                payload, inv, _ = ops.fp8_quantize(w.detach())
            cached = (key, payload, inv.reshape(1))
            self._fp8_cache = cached
        return cached[1], cached[2]

    def _weight_fp8_transposed(self, w8):
        """The [K,N] copy of the cached weight payload `w8` (the operand of grad_input), made once per weight version."""
        cached = getattr(self, "_fp8_cache_t", None)
        if cached is None or cached[0] is not w8:
            cached = (w8, ops.fp8_transpose(w8))
            self._fp8_cache_t = cached
        return cached[1]

    def forward(self, input):
        if not input.is_cuda:
            raise RuntimeError("Float8Linear runs on the GPU only; there is no CPU fallback")
        input = input.to(torch.bfloat16 if COMPUTE_DTYPE == torch.float32 else COMPUTE_DTYPE)
        if input.dtype != torch.bfloat16:
            raise ValueError("Float8Linear: the GPU path computes in bf16")
        orig_shape = input.shape
        x2 = input.reshape(-1, orig_shape[-1])
        if torch.is_grad_enabled() and (x2.requires_grad or self.weight.requires_grad):
            out = _Float8Matmul.apply(x2, self.weight, self)
        else:
            a8, inv_a, _ = ops.fp8_quantize(x2)
            w8, inv_w = self._weight_fp8()
            out = ops.fp8_gemm(a8, w8, inv_a, inv_w)
        out = out.reshape(*orig_shape[:-1], out.shape[-1])
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out

    @classmethod
    def from_float(cls, mod):
        """Shell on the meta device that shares mod's weight and bias (fp8.py:215-227)."""
        with torch.device("meta"):
            new = cls(mod.in_features, mod.out_features, bias=False)
        new.weight = mod.weight
        new.bias = mod.bias
        return new


class Float8LinearConfig:
    """Only the tensorwise recipe exists (fp8.py:230-240)."""

    @staticmethod
    def from_recipe_name(recipe_name):
        if recipe_name != "tensorwise":
            raise ValueError(f"Only 'tensorwise' recipe is supported, got '{recipe_name}'. "
                             f"Rowwise/axiswise recipes require the full torchao library.")
        return Float8LinearConfig()


def fp8_module_filter(mod, fqn=""):
    """The filter the reference trains with (scripts/base_train.py:178-185)."""
    if not isinstance(mod, nn.Linear):
        return False
    if mod.in_features % 16 != 0 or mod.out_features % 16 != 0:
        return False
    return min(mod.in_features, mod.out_features) >= 128


def convert_to_float8_training(module, *, config=None, module_filter_fn=None):
    """Swap nn.Linear children for Float8Linear, children first (fp8.py:243-266)."""
    def walk(mod, prefix=""):
        for name, child in list(mod.named_children()):
            fqn = f"{prefix}.{name}" if prefix else name
            walk(child, fqn)
            if isinstance(child, nn.Linear) and not isinstance(child, Float8Linear):
                if module_filter_fn is None or module_filter_fn(child, fqn):
                    setattr(mod, name, Float8Linear.from_float(child))
    walk(module)
    if hasattr(module, "invalidate_plan"):      # a model that caches quantized weights per module starts over
        module.invalidate_plan()
    return module
