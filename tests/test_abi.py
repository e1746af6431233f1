"""The C-ABI library loads and exports every function the public header declares (no GPU needed)."""
import ctypes
import os
import re

from nanochat_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "nanochat_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nc_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_functions()
    assert len(names) >= 16
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/nanochat_amd.h but not exported"
    assert sorted(_lib.EXPORTS) == names


def test_binding_and_error_channel():
    lib = _lib.lib()
    assert lib.nc_abi_version() == 1
    # argument validation happens before any GPU call, so it can be exercised without a device
    rc = lib.nc_fp8_quantize_tensorwise(None, 0, 16, None, None, None, None, 0, None)
    assert rc == -1 and b"null pointer" in lib.nc_last_error()
    rc = lib.nc_fp8_gemm_tn(None, None, None, None, None, 1, None, 0, 0.0, 4, 4, 16, 4, 0, None, 0, None)
    assert rc == -1
    rc = lib.nc_sample(None, 1, 8, 8, 1.0, 0, None, None, None)
    assert rc == -1


def test_struct_layout_matches_header():
    # pointer-sized fields + ints: sizes as a C compiler lays them out on LP64
    assert ctypes.sizeof(_lib.LayerDesc) == 10 * 8 + 2 * 4
    assert ctypes.sizeof(_lib.ModelDesc) == 8 * 4 + 2 * 4 + 11 * 8
    assert ctypes.sizeof(_lib.CacheDesc) == 5 * 8 + 2 * 4
