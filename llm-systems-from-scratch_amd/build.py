"""Builds libmi355attn.so (the C-ABI HIP library) for gfx950 with hipcc.

Usage: python build.py            (from anywhere; output lands next to the
Python package so the built library travels with the source tree)
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "mi355_attn")
LIB_NAME = "libmi355attn.so"
SOURCES = ["api.hip", "paged_decode.hip", "prefill_fwd.hip", "prefill_fwd_w64.hip", "prefill_bwd.hip", "kv_cache_ops.hip",
           "layer_ops.hip"]
# prefill_fwd_w64.hip keeps its output accumulators in AGPRs that only its assembly statements touch: its builtin MFMAs
# must therefore be selected in VGPR form, so that the compiler allocates no AGPR for them.
# It is also compiled without the machine-code hoisting of loop invariants: hoisted out of the job loop, a few dozen
# per-lane addresses stayed live across the assembly loop (which owns most vector registers) and pushed the
# prefetched query rows into scratch memory, whose reloads wait for every load in flight.
EXTRA_FLAGS = {"prefill_fwd_w64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-disable-machine-licm"]}

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-fno-gpu-rdc", "-Wall", "-Wno-unused-function",
    # packed-fp32 VALU forms are kept off for every device pass
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def library_path() -> str:
    return os.path.join(OUT_DIR, LIB_NAME)


def build_library(verbose: bool = True) -> str:
    # the hand-scheduled assembly of prefill_fwd_w64.hip is generated text: regenerate it so that it cannot go stale
    _run([sys.executable, os.path.join(CSRC, "gen_prefill_w64_loop.py")])
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(src):
        obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
        log = _run([HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj])
        return obj, log

    with ThreadPoolExecutor(max_workers=4) as ex:
        results = list(ex.map(compile_one, srcs))
    for _, log in results:
        if verbose and log.strip():
            print(log)
    lib = library_path()
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *[o for o, _ in results]])
    if verbose:
        print("built", lib)
    return lib


if __name__ == "__main__":
    build_library()
    sys.exit(0)
