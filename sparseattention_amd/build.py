"""Build libsparseattn_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: ``python -m sparseattention_amd.build`` or :func:`build_library`.
The library is written next to this file so that it is found in-tree.
"""
from __future__ import annotations

import os
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
         ("fwd_schedule.hip", "fwd_schedule.o", []), ("sparse_fwd.hip", "sparse_fwd.o", []),
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
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libsparseattn_hip.so cannot be built")
    return exe


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + r.stdout + r.stderr)
    # the host pass does not know the AMDGPU feature name and says so; everything else is shown
    noise = "is not a recognized feature for this target"
    out = "\n".join(line for line in (r.stdout + r.stderr).splitlines() if noise not in line).strip()
    if out:
        print(out, file=sys.stderr)


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
