"""Builds the C part of the oracle (test infrastructure only).

    python -m oracle.build_oracle

Output goes to oracle/_build/libe4m3_oracle.so.  The reference is pure Python, so
there is no reference build to make (no oracle/_ref).
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
OUT_DIR = os.path.join(HERE, "_build")
LIB = os.path.join(OUT_DIR, "libe4m3_oracle.so")


def build(force=True):
    os.makedirs(OUT_DIR, exist_ok=True)
    if force or not os.path.exists(LIB):
        cmd = ["gcc", "-O2", "-shared", "-fPIC", "-ffp-contract=off", "-o", LIB,
               os.path.join(HERE, "e4m3.c"), "-lm"]
        subprocess.run(cmd, check=True)
    return LIB


def load():
    """ctypes handle to the C oracle, building it if it is missing."""
    import ctypes
    lib = ctypes.CDLL(build(force=False))
    c = ctypes
    lib.oracle_e4m3_encode.restype = c.c_uint8
    lib.oracle_e4m3_encode.argtypes = [c.c_float]
    lib.oracle_e4m3_decode.restype = c.c_float
    lib.oracle_e4m3_decode.argtypes = [c.c_uint8]
    for name in ("oracle_quantize_f32", "oracle_quantize_bf16"):
        fn = getattr(lib, name)
        fn.restype = None
        fn.argtypes = [c.c_void_p, c.c_size_t, c.c_void_p, c.c_void_p, c.c_void_p]
    lib.oracle_encode_bf16_with_scale.restype = None
    lib.oracle_encode_bf16_with_scale.argtypes = [c.c_void_p, c.c_size_t, c.c_float, c.c_void_p]
    return lib


if __name__ == "__main__":
    print(build())
