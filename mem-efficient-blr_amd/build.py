"""Build libblr.so (the HIP kernels and their C ABI) for gfx950, in-tree.

    python build.py            # -> lib/libblr.so next to this file

Plain hipcc, no build system.  Objects are compiled in parallel, then linked.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = ["blr_api.hip", "blr_gemm.hip", "blr_stream.hip", "blr_decode.hip", "blr_decode3.hip", "blr_decode_pair.hip", "blr_decode_rows.hip", "blr_prefill.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wno-pass-failed", "-Wno-unused-function"]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 target feature and says so; that is harmless
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError(f"{' '.join(cmd)}\n{out}")
    return out


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    if not os.path.exists(hipcc):
        hipcc = "hipcc"
    os.makedirs(os.path.join(HERE, "lib"), exist_ok=True)
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    objs = []

    def compile_one(name):
        obj = os.path.join(HERE, "build", name.replace(".hip", ".o"))
        out = _run([hipcc, *FLAGS, "-c", os.path.join(HERE, "csrc", name), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=len(SRC)) as ex:
        objs = list(ex.map(compile_one, SRC))
    so = os.path.join(HERE, "lib", "libblr.so")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", so])
    if verbose:
        print(f"built {so}")
    return so


if __name__ == "__main__":
    try:
        build()
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
