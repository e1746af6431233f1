"""Compute dtype selection and hardware peak tables (nanochat/common.py:16-32, 228-328)."""
import os

import torch

_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


def _detect_compute_dtype():
    """NANOCHAT_DTYPE wins; a GPU means bf16; no GPU means fp32 (common.py:16-32)."""
    env = os.environ.get("NANOCHAT_DTYPE")
    if env is not None:
        return _DTYPES[env]
    return torch.bfloat16 if torch.cuda.is_available() else torch.float32


COMPUTE_DTYPE = _detect_compute_dtype()

# Dense peaks of one MI355X.  bf16 and HBM are the values of common.py:258 and :311; the fp8 figure is
# twice the bf16 one (full-rate f8f6f4 MFMA).
PEAK_BF16_FLOPS = 2.5e15
PEAK_FP8_FLOPS = 5.0e15
PEAK_HBM_BYTES_PER_S = 8.0e12


def get_peak_flops(device_name=None):
    """Dense bf16 peak (common.py:228-270).  The library's kernels exist for gfx950 only, so there is one answer whatever the driver
    calls the device (some report an empty or generic name); the argument is kept for the reference's signature."""
    return PEAK_BF16_FLOPS


def get_peak_bandwidth(device_name=None):
    """HBM peak (common.py:300-328); one answer, as for get_peak_flops."""
    return PEAK_HBM_BYTES_PER_S


def print0(*args, **kwargs):
    if int(os.environ.get("RANK", 0)) == 0:
        print(*args, **kwargs)
