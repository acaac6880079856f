"""Build recipe of the HIP library: ``python sglang-jax_amd/build.py``.

Compiles every translation unit under ``csrc/`` for gfx950 with hipcc (it
cross-compiles without a GPU) and links ``lib/librpa_mi355.so`` in-tree.
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(OUT_DIR, "librpa_mi355.so")
HASH_PATH = os.path.join(OUT_DIR, "librpa_mi355.srchash")

SOURCES = ["rpa_capi.hip", "rpa_decode.hip", "rpa_prefill.hip", "rpa_prefill_pipe.hip", "rpa_mla.hip"]
# bench.py's measurement kernels (a streaming read, a matrix-instruction issue loop): a library of their own,
# so that the attention library carries nothing but the attention path
CEILINGS_SOURCE = "rpa_ceilings.hip"
CEILINGS_LIB_PATH = os.path.join(OUT_DIR, "librpa_ceilings.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-fPIC",
    "-std=c++17",
    "-ffp-contract=fast",
    # only the RPA_API entry points of include/rpa.h are dynamic symbols
    "-fvisibility=hidden",
    "-fvisibility-inlines-hidden",
    # never let the compiler form packed-fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-inline-asm",  # async_copy16 names m0, which the compiler reports as reserved
]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    noise = ("is not a recognized feature for this target",)
    out = "\n".join(ln for ln in proc.stdout.splitlines() if not any(n in ln for n in noise))
    return out


def source_hash() -> str:
    """Hash of everything the library is compiled from (and of the flags)."""
    import hashlib

    h = hashlib.sha256(" ".join(FLAGS).encode())
    files = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if os.path.isfile(os.path.join(CSRC, f)))
    files.append(os.path.join(os.path.dirname(HERE), "include", "rpa.h"))
    for path in files:
        h.update(os.path.basename(path).encode())
        with open(path, "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def build(verbose: bool = False, extra_flags=()) -> str:
    os.makedirs(OUT_DIR, exist_ok=True)
    objs = []

    def compile_one(src):
        obj = os.path.join(OUT_DIR, src.replace(".hip", ".o"))
        out = _run([HIPCC, *FLAGS, *extra_flags, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(compile_one, SOURCES + [CEILINGS_SOURCE]))
    ceil_obj = objs.pop()
    for path, members in ((LIB_PATH, objs), (CEILINGS_LIB_PATH, [ceil_obj])):
        tmp = path + ".tmp"
        _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *members, "-o", tmp])
        os.replace(tmp, path)
    objs.append(ceil_obj)
    if not extra_flags:
        with open(HASH_PATH, "w") as f:
            f.write(source_hash() + "\n")
    elif os.path.exists(HASH_PATH):
        os.remove(HASH_PATH)  # an experimental build never passes for the committed sources
    for o in objs:
        os.remove(o)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose=True, extra_flags=sys.argv[1:])
    print("built", path)
