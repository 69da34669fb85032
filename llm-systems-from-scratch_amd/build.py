"""Builds libmi355attn.so (the C-ABI HIP library) for gfx950 with hipcc.

Usage: python build.py            (from anywhere; output lands next to the
Python package so the built library travels with the source tree)
"""
from __future__ import annotations

import os
import re
import subprocess
import sys
import tempfile
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
EXTRA_FLAGS = {"prefill_fwd_w64.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1", "-mllvm", "-disable-machine-licm"],
               # prefill_bwd.hip orders its LDS reads and MFMAs by hand (reads two MFMAs ahead, a scheduling barrier after
               # every MFMA); the scheduler that runs after register allocation undoes part of that: 1.5 % (measured)
               "prefill_bwd.hip": ["-mllvm", "-enable-post-misched=0"]}

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


def check_w64_registers() -> str:
    """prefill_fwd_w64.hip keeps values in a[0:N_AGPRS-1] across its assembly statements, behind the compiler's back:
    the statements name those registers as clobbered, so the compiler holds nothing of its own in them ACROSS a
    statement, but nothing in the language keeps it from using one BETWEEN two statements (as a spill slot, say).
    This compiles the file to assembly and fails the build if any instruction outside the statements touches one."""
    n_agprs = 0
    with open(os.path.join(CSRC, "prefill_w64_asm.inc")) as f:
        for line in f:
            if line.startswith("#define W64_CLOBBER_ACC"):
                n_agprs = line.count('"a')
    if n_agprs == 0:
        raise RuntimeError("prefill_w64_asm.inc: no W64_CLOBBER_ACC")
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "w64.s")
        _run([HIPCC, *FLAGS, *EXTRA_FLAGS["prefill_fwd_w64.hip"], "-S", "--cuda-device-only",
              os.path.join(CSRC, "prefill_fwd_w64.hip"), "-o", asm])
        inside, bad = False, []
        with open(asm) as f:
            for no, line in enumerate(f, 1):
                if "#ASMSTART" in line:
                    inside = True
                elif "#ASMEND" in line:
                    inside = False
                elif not inside and not line.lstrip().startswith((";", ".")):
                    for m in re.finditer(r"\ba\[(\d+):\d+\]|\ba(\d+)\b", line.split(";")[0]):
                        if int(m.group(1) or m.group(2)) < n_agprs:
                            bad.append("%d: %s" % (no, line.strip()))
        if bad:
            raise RuntimeError("prefill_fwd_w64.hip: compiler-generated code touches AGPRs below a%d, which the "
                               "assembly statements own:\n%s" % (n_agprs, "\n".join(bad[:20])))
    return "prefill_fwd_w64.hip: no compiler-generated instruction touches a[0:%d]" % (n_agprs - 1)


_SREG = re.compile(r"\bs\[(\d+):(\d+)\]|\bs(\d+)\b")


def _sregs(text):
    out = set()
    for m in _SREG.finditer(text):
        if m.group(3) is not None:
            out.add(int(m.group(3)))
        else:
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
    return out


def check_scalar_address_hazards(src: str) -> str:
    """gfx9 wants five wait states between a VECTOR instruction that writes a scalar register (v_readlane restoring a
    spilled value, v_readfirstlane, a compare or a carry-out) and a vector-memory instruction that reads that register
    as its address.  The compiler inserts them for the instructions it emits, but it cannot see inside an
    inline-assembly statement, and the direct-to-LDS loads of these kernels live in such statements.  This compiles
    `src` to assembly and fails the build if a memory instruction inside a statement reads a scalar register that a
    vector instruction wrote fewer than five wait states earlier on the straight-line path in front of it."""
    with tempfile.TemporaryDirectory() as tmp:
        asm = os.path.join(tmp, "k.s")
        _run([HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", asm])
        lines = open(asm).read().splitlines()
    bad, inside, n_checked = [], False, 0
    code = []                     # (line number, text) of instructions, in order
    for no, raw in enumerate(lines, 1):
        text = raw.split(";")[0].strip()
        if "#ASMSTART" in raw:
            inside = True
            continue
        if "#ASMEND" in raw:
            inside = False
            continue
        if not text or text.startswith(".") or text.endswith(":"):
            continue
        code.append((no, text, inside))
    for i, (no, text, in_asm) in enumerate(code):
        op = text.split()[0]
        if not in_asm or not op.startswith(("global_", "buffer_", "flat_", "scratch_")):
            continue
        addr = _sregs(text)
        if not addr:
            continue
        n_checked += 1
        states, j = 0, i - 1
        while j >= 0 and states < 5:
            _, prev, _ = code[j]
            pop = prev.split()[0]
            if pop == "s_nop":
                states += int(prev.split()[1], 0) + 1
            else:
                # destination operands of a vector instruction: everything in front of the first source; an SGPR
                # there (v_readlane sN, v_cmp_* s[a:b], the carry-out of v_mad_u64_u32 / v_add_co) is a vector write
                if pop.startswith("v_"):
                    ops = prev[len(pop):].split(",")
                    n_dst = 2 if pop.startswith(("v_mad_u64", "v_mad_i64", "v_add_co", "v_sub_co", "v_addc", "v_subb",
                                                  "v_div_scale")) else 1
                    written = set()
                    for o in ops[:n_dst]:
                        written |= _sregs(o)
                    if written & addr:
                        bad.append("%s:%d: `%s` reads s%s, written %d wait state(s) earlier by `%s`"
                                   % (src, no, text, sorted(written & addr), states, prev))
                        break
                states += 1
            j -= 1
    if bad:
        raise RuntimeError("scalar address hazard in inline assembly:\n" + "\n".join(bad[:20]))
    return "%s: %d inline-assembly memory instructions, none reads a scalar register within five wait states of a vector write" % (src, n_checked)


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

    # sources whose kernels issue memory instructions from inline assembly
    asm_dma = [s for s in ("prefill_fwd.hip", "prefill_fwd_w64.hip", "prefill_bwd.hip") if s in srcs]
    with ThreadPoolExecutor(max_workers=4) as ex:
        check = ex.submit(check_w64_registers)
        hazards = [ex.submit(check_scalar_address_hazards, s) for s in asm_dma]
        results = list(ex.map(compile_one, srcs))
        notes = [check.result()] + [h.result() for h in hazards]
    if verbose:
        print("\n".join(notes))
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
