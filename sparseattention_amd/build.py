"""Build libsparseattn_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: ``python -m sparseattention_amd.build`` or :func:`build_library`.
The library is written next to this file so that it is found in-tree.
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
CSRC = os.path.join(_HERE, "csrc")
INCLUDE = os.path.join(_ROOT, "include")
LIB_PATH = os.path.join(_HERE, "libsparseattn_hip.so")

# (source, object name, extra defines).  The forward kernels are one source compiled per element type and
# mask source, so that the variants build in parallel.
UNITS = [("sparseattn_api.hip", "sparseattn_api.o", []), ("mask_classify.hip", "mask_classify.o", []),
         ("mask_terms.hip", "mask_terms.o", []),
         ("fwd_schedule.hip", "fwd_schedule.o", []), ("sparse_fwd.hip", "sparse_fwd.o", []),
         ("sparse_fwd_f32.hip", "sparse_fwd_f32.o", []), ("sparse_fwd_c32.hip", "sparse_fwd_c32.o", []),
         ("sparse_fwd_f32_mfma.hip", "sparse_fwd_f32_mfma.o", []),
         ("sparse_decode.hip", "sparse_decode.o", []), ("sparse_bwd.hip", "sparse_bwd.o", [])]
UNITS += [("sparse_fwd_inst.hip", f"sparse_fwd_dt{dt}_pk{pk}_ps{ps}.o",
           [f"-DSA_FWD_DT={dt}", f"-DSA_FWD_PK={pk}", f"-DSA_FWD_PS={ps}"])
          for dt in (0, 1) for pk in (0, 1) for ps in (0, 1)]

# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32 from float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-command-line-argument",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Rpass-analysis=kernel-resource-usage",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libsparseattn_hip.so cannot be built")
    return exe


def kernel_resources(remarks: str) -> dict:
    """{kernel symbol: {"VGPRs": n, "ScratchSize": n, ...}} from the compiler's kernel-resource-usage remarks."""
    found, name = {}, None
    for line in remarks.splitlines():
        m = re.search(r"remark:\s+Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            found[name] = {}
            continue
        m = re.search(r"remark:\s+([A-Za-z ]+?)(?: \[[^\]]*\])?: (\d+|True|False) \[-Rpass-analysis", line)
        if m and name is not None:
            found[name][m.group(1).replace(" ", "")] = int({"True": 1, "False": 0}.get(m.group(2), m.group(2)))
    return found


# The most vector registers a kernel may spill (the scheduled forward with bool-mask reads at D = 128 spills 6-8 of
# its 256, which costs it about 1 %).
MAX_SPILLED_VGPRS = 8


def scratch_offenders(resources: dict) -> dict:
    """The kernels of :func:`kernel_resources` output that must not ship.

    Every kernel of this library keeps its state in registers.  One whose arrays the compiler could not split into
    registers (scratch memory without spilled registers: a variable index into a small array is enough) runs several
    times slower with the same results, which no parity test would notice; so does one that spills many registers
    to scratch memory (registers "spilled" without any scratch went to the other half of the register file of a
    kernel that runs one wave per SIMD, which is no concern).
    """
    return {k: v for k, v in resources.items()
            if v.get("DynamicStack", 0)
            or (v.get("ScratchSize", 0) and not 0 < v.get("VGPRsSpill", 0) <= MAX_SPILLED_VGPRS)}


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    text = r.stdout + r.stderr
    res = kernel_resources(text)
    bad = scratch_offenders(res)
    if bad:
        raise RuntimeError("kernels using scratch memory in " + " ".join(cmd[-3:]) + ": " +
                           ", ".join(f"{k} ({v.get('ScratchSize', 0)} bytes/lane, {v.get('VGPRsSpill', 0)} spilled registers)"
                                     for k, v in bad.items()))
    # the host pass does not know the AMDGPU feature name and says so; the resource remarks were read above, their
    # source excerpts ("  54 | __global__ ...", "     | ^") go with them; everything else is shown
    noise = ("is not a recognized feature for this target", "-Rpass-analysis=kernel-resource-usage")
    lines = [ln for ln in text.splitlines() if not any(n in ln for n in noise)]
    lines = [ln for ln in lines if not re.match(r"^\s*\d*\s*\|", ln)]
    out = "\n".join(lines).strip()
    if out and re.search(r"(warning|error|note):", out):  # else only the include trails of the remarks are left
        print(out, file=sys.stderr)
    return res


def build_library(verbose: bool = False, extra_flags=()) -> str:
    """Compile every kernel translation unit and link the shared library.  Always recompiles."""
    hipcc = _hipcc()
    obj_dir = os.path.join(_HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, o) for _, o, _ in UNITS]
    cmds = [[hipcc, *HIPCC_FLAGS, *extra_flags, *defs, "-c", os.path.join(CSRC, src), "-o", obj]
            for (src, _, defs), obj in zip(UNITS, objs)]
    if verbose:
        for c in cmds:
            print(" ".join(c))
    with ThreadPoolExecutor(max_workers=min(os.cpu_count() or 4, len(cmds), 8)) as ex:
        list(ex.map(_run, cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc", *objs, "-o", LIB_PATH])
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
