"""Builds the HIP library in-tree (``orangu_amd/liborangu_mi355x.so``) for gfx950.

hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is installed.
"""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "liborangu_mi355x.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

SOURCES = ["ogm_kernels.hip", "ogm_gemm.hip", "ogm_gemm_ft.hip", "ogm_llama.hip", "ogm_static.hip", "ogm_api.cpp", "ogm_repack.cpp", "ogm_gguf.cpp"]

# -ffp-contract=off: the kernels reproduce the CPU path's f32 results bit for bit, which an FMA
#   contraction would break.
# -packed-fp32-ops off: keeps hipcc from forming packed FP32 instructions out of scalar code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # scalar and pointer arguments at the front of a kernel's argument list arrive in SGPRs with the wave instead of
    # behind a scalar load at its start (gfx940 and later): 0.6 % of a decode step of 257 dependent launches
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


# Flags for single files.  ogm_gemm_ft.hip: its matrix instructions' results feed vector instructions at
# once; kept in vector registers they need no copies out of the accumulation registers.
EXTRA_FLAGS = {"ogm_gemm_ft.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def build(verbose: bool = False, defines=(), out: str | None = None) -> str:
    """Compiles every source to an object of its own (in parallel) and links the shared library.
    `defines` (NAME=VALUE strings, passed as -D) and `out` build a variant beside the library instead of it: the
    kernels' timing switches (GD_ABL_*, SBW_ABL, FK_ABL: wrong results, for `bench.py --lib`)."""
    from concurrent.futures import ThreadPoolExecutor
    names = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    if defines and not out:
        raise ValueError("a build with defines needs an output path of its own")
    lib_path = os.path.abspath(out) if out else LIB_PATH
    obj_dir = os.path.join(HERE, "build") if not out else lib_path + ".objs"
    os.makedirs(obj_dir, exist_ok=True)
    dflags = ["-D" + d for d in defines]
    noise = "is not a recognized feature for this target"

    def run(cmd):
        proc = subprocess.run(cmd, capture_output=True, text=True)
        log = "\n".join(l for l in (proc.stdout + proc.stderr).splitlines() if noise not in l)
        if proc.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + log)
        return log

    def compile_one(name):
        obj = os.path.join(obj_dir, name + ".o")
        return obj, run([hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(name, []), *dflags, "-c", os.path.join(CSRC, name), "-o", obj])

    with ThreadPoolExecutor(max_workers=min(8, len(names))) as pool:
        done = list(pool.map(compile_one, names))
    log = "\n".join(l for _, l in done if l.strip())
    log += run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path, *[o for o, _ in done]])
    if out:
        shutil.rmtree(obj_dir, ignore_errors=True)
    if verbose and log.strip():
        print(log)
    return lib_path


if __name__ == "__main__":
    import argparse
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--define", action="append", default=[], metavar="NAME=VALUE",
                    help="a timing switch of the kernels (-DNAME=VALUE); needs --out")
    ap.add_argument("--out", default=None, help="write the library here instead of in-tree")
    a = ap.parse_args()
    print(build(verbose=True, defines=a.define, out=a.out))
