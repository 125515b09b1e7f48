"""Compile libctmi.so (HIP, gfx950) in-tree with hipcc.

    python -m compressed_tensors_amd._build        # or  build_library()

hipcc cross-compiles for gfx950 without a GPU.  The library lands next to this
file (lib/libctmi.so); it is git-ignored but travels with the source tree.
"""
import os
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR.parent / "csrc"
INCLUDE_DIR = PKG_DIR.parent.parent / "include"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libctmi.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # correctly rounded fp32 division and no contraction: results must match torch bit for bit
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-ffp-contract=off",
    "-fno-fast-math",
    # do not let the compiler form packed-fp32 instructions
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
]


# per source file (by stem): the butterfly kernels and the rotations with an epilogue chain
# matrix-core results into vector code, so their accumulators live in ordinary registers (no
# copies out of a second register class - one instruction per output element -, and the
# registers are reused once the accumulators are dead)
EXTRA_FLAGS = {"fwht": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
               "hadamard": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}


def sources():
    return sorted(str(p) for p in CSRC_DIR.glob("*.hip"))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build_library(verbose: bool = False, jobs: int = 0) -> Path:
    """compile every source file (one hipcc process each, `jobs` at a time) and link"""
    from concurrent.futures import ThreadPoolExecutor

    LIB_DIR.mkdir(parents=True, exist_ok=True)
    obj_dir = LIB_DIR / "obj"
    obj_dir.mkdir(exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"]
    srcs = sources()
    objs = [str(obj_dir / (Path(src).stem + ".o")) for src in srcs]
    jobs = jobs or min(len(srcs), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(
            lambda so: _run([HIPCC, *compile_flags, *EXTRA_FLAGS.get(Path(so[0]).stem, []),
                             f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}", "-c", so[0], "-o", so[1]], verbose),
            zip(srcs, objs)))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)], verbose)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
