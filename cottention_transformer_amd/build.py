"""Builds libcottention_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

    python -m cottention_transformer_amd.build            # compile every translation unit and link
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build", "obj")
LIB_PATH = os.path.join(HERE, "lib", "libcottention_hip.so")

SOURCES = ["cott_api.hip", "cott_mfma_bf16.hip", "cott_mfma_fp16.hip", "cott_mfma_f32.hip", "cott_generic.hip", "cott_prep.hip", "cott_calib.hip"]

# -packed-fp32-ops off: scalar/float2 fp32 code must not be fused into v_pk_*_f32 instructions.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc()] + HIPCC_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    return obj, out


def build(verbose=False, jobs=None):
    """Compile all HIP sources and link the shared library; returns its path."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(os.path.dirname(LIB_PATH), exist_ok=True)
    jobs = jobs or min(len(SOURCES), max(1, (os.cpu_count() or 2) // 2))
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(_compile, SOURCES))
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    objs = [o for o, _ in results]
    tmp = LIB_PATH + ".tmp"
    link = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs
    res = subprocess.run(link, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stdout)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
