"""Build libblr.so (the HIP kernels and their C ABI) for gfx950, in-tree, and the stand-alone probes under probes/.

    python build.py            # -> lib/libblr.so next to this file, probes/<name> next to probes/<name>.hip

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
    # the stand-alone probes (not part of the library): built next to their sources so that they compile as long as the tree does
    probes = [n[:-4] for n in sorted(os.listdir(os.path.join(HERE, "probes"))) if n.endswith(".hip")]
    with ThreadPoolExecutor(max_workers=max(1, len(probes))) as ex:
        list(ex.map(lambda n: _run([hipcc, *[f for f in FLAGS if f != "-fPIC"], os.path.join(HERE, "probes", n + ".hip"), "-o",
                                    os.path.join(HERE, "probes", n)]), probes))
    if verbose and probes:
        print("built probes:", ", ".join(probes))
    return so


if __name__ == "__main__":
    try:
        build()
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
