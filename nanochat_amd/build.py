"""Builds libnanochat_amd.so for gfx950 with hipcc (no torch headers, no cmake).

    python -m nanochat_amd.build

The library is written next to this file so it travels with the source tree.
"""
import hashlib
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "_build")
LIB_PATH = os.path.join(HERE, "libnanochat_amd.so")
STAMP_PATH = LIB_PATH + ".sources"           # digest of what the library was built from

SOURCES = ["nc_api.hip", "nc_quantize.hip", "nc_gemm.hip", "nc_elementwise.hip", "nc_attention.hip", "nc_attention_prefill.hip",
           "nc_sample.hip", "nc_forward.hip", "nc_profile.hip", "nc_gemm_decode.hip"]

# -packed-fp32-ops off: packed fp32 VALU forms are not to be generated on this hardware pool
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def sources_digest():
    """SHA-256 over the flags and every file the library is compiled from."""
    h = hashlib.sha256(" ".join(FLAGS).encode())
    files = [os.path.join(CSRC, f) for f in sorted(os.listdir(CSRC)) if f.endswith((".hip", ".h"))]
    files.append(os.path.join(os.path.dirname(HERE), "include", "nanochat_amd.h"))
    for f in files:
        h.update(os.path.basename(f).encode())
        h.update(open(f, "rb").read())
    return h.hexdigest()


def _compile(src):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    cmd = ["hipcc", *FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    return src, obj, r


def build(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    if os.path.exists(STAMP_PATH):
        os.remove(STAMP_PATH)              # a failed build must not leave a stamp that matches
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = []
    for src, obj, r in results:
        noise = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stderr}")
        if verbose and noise:
            print(f"[{src}]\n" + "\n".join(noise), file=sys.stderr)
        objs.append(obj)
    link = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    r = subprocess.run(link, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr}")
    with open(STAMP_PATH, "w") as f:
        f.write(sources_digest() + "\n")
    return LIB_PATH


if __name__ == "__main__":
    print(build())
