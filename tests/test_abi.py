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
    assert lib.nc_abi_version() == 2
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
    assert ctypes.sizeof(_lib.CacheDesc) == 5 * 8 + 5 * 4 + 4


def test_library_was_built_from_these_sources():
    """A failed rebuild leaves the previous library in place; tests must not pass against a stale one.  The build writes the
    digest of its inputs next to the library."""
    from nanochat_amd import build as nb
    assert os.path.exists(nb.STAMP_PATH), "no build stamp next to the library: run python -m nanochat_amd.build"
    assert open(nb.STAMP_PATH).read().strip() == nb.sources_digest(), \
        "nanochat_amd/libnanochat_amd.so was built from other sources than the tree holds: run python -m nanochat_amd.build"


def test_hot_kernels_use_no_scratch_memory():
    """The streaming kernels keep their state in registers: a private-memory spill costs the decode attention 15 %.
    Compiles the sources that hold them with the resource-usage remarks on and reads the figures."""
    import subprocess
    from nanochat_amd import build as nb
    # bytes of scratch per lane allowed: the persistent GEMM keeps a few tile-level addresses there (outside its K loop); the
    # attention variants with 4 or 8 query heads per kv head reserve 20 bytes for a spilled scalar register's lane store and
    # touch them with no instruction
    hot = {"nc_attention.hip": {"attn_partial_kernel": 32},
           "nc_gemm_decode.hip": {"gemm_decode_kernel": 0, "finish_partials_kernel": 0},
           "nc_elementwise.hip": {"mix_norm_vec_kernel": 0, "kv_prefill_copy_kernel": 0, "qkv_rope_append_kernel": 0},
           "nc_gemm.hip": {"gemm_dl_kernel": 0, "gemm_dlp_kernel": 64},
           "nc_attention_prefill.hip": {"attn_prefill_kernel": 0},
           "nc_quantize.hip": {"amax_kernel": 0, "convert_kernel": 0, "transpose_u8_kernel": 0},
           "nc_sample.hip": {"sample_kernel": 0}}
    for src, kernels in hot.items():
        cmd = ["hipcc", *nb.FLAGS, "-Rpass-analysis=kernel-resource-usage", "-c", os.path.join(nb.CSRC, src), "-o", os.devnull]
        r = subprocess.run(cmd, capture_output=True, text=True)
        assert r.returncode == 0, r.stderr[-2000:]
        name, seen = None, set()
        for line in r.stderr.splitlines():
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                name = m.group(1)
            m = re.search(r"ScratchSize \[bytes/lane\]: (\d+)", line)
            if m and name:
                for k in kernels:
                    if k in name:
                        seen.add(k)
                        assert int(m.group(1)) <= kernels[k], f"{name} in {src} uses {m.group(1)} bytes of scratch per lane"
        assert seen == set(kernels), f"{src}: kernels not found in the compiler's report: {set(kernels) - seen}"
