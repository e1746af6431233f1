"""Float8Linear on MI355X: tensorwise e4m3 quantization + FP8 MFMA GEMM, forward only.

Same public surface as nanochat/fp8.py (Float8Linear :195-227, Float8LinearConfig :230-240,
convert_to_float8_training :243-266).  Differences that do not change results:
  * the weight is quantized once and kept (payload + inverse scale) until the parameter's storage or
    version counter changes; the reference re-quantizes it on every call (fp8.py:136), which for a
    frozen weight produces the same bytes;
  * there is no backward: this is the inference path.
"""
import torch
import torch.nn as nn

from . import ops
from .common import COMPUTE_DTYPE


class Float8Linear(nn.Linear):
    """nn.Linear whose matmul runs in FP8 on the GPU (fp8.py:195-213)."""

    def _weight_fp8(self):
        w = self.weight
        key = (w.data_ptr(), w._version, w.dtype, tuple(w.shape))
        cached = getattr(self, "_fp8_cache", None)
        if cached is None or cached[0] != key:
            payload, inv, _ = ops.fp8_quantize(w.detach())
            cached = (key, payload, inv.reshape(1))
            self._fp8_cache = cached
        return cached[1], cached[2]

    @torch.no_grad()
    def forward(self, input):
        if not input.is_cuda:
            raise RuntimeError("Float8Linear runs on the GPU only; there is no CPU fallback")
        input = input.to(torch.bfloat16 if COMPUTE_DTYPE == torch.float32 else COMPUTE_DTYPE)
        if input.dtype != torch.bfloat16:
            raise ValueError("Float8Linear: the GPU path computes in bf16")
        orig_shape = input.shape
        x2 = input.reshape(-1, orig_shape[-1])
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
    return module
