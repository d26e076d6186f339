"""Build the gfx950 shared library in-tree with hipcc.

``python -m trifast_amd.build`` compiles every ``csrc/*.hip`` translation unit for
``--offload-arch=gfx950`` (in parallel) and links ``trifast_amd/libtrifast_hip.so``.
hipcc cross-compiles without a GPU, so this runs anywhere the ROCm toolchain is.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "libtrifast_hip.so"
LIB_PATH = PKG_DIR / LIB_NAME

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    # keep MFMA accumulators in VGPRs: no accvgpr copies around the softmax math
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # (m0 is set by hand around the global->LDS loads written as asm)
    "-Wno-inline-asm",
]


# per-source additions, measured on MI355X: the db kernel (4 waves per SIMD, short
# dependent chains per row) runs 3-4 % faster when scheduled for instruction-level
# parallelism; the other kernels are better off with the default strategy
PER_SOURCE_FLAGS = {
    "tri_bwd_b.hip": ["-mllvm", "-amdgpu-sched-strategy=max-ilp"],
}


# The row-resident backward issues some of its MFMAs from asm statements with hand-placed wait
# states (csrc/tri_common.hpp: mfma_acc).  That schedule was validated, by the parity and
# bit-equality tests of the row-resident kernel, with the compiler named here; any other one
# builds those MFMAs through the compiler's own intrinsic instead (slower where the register
# file is full, but hazard-free by construction) and says so.
VALIDATED_COMPILER = "roc-7.2.0"


def _compiler_flags() -> list[str]:
    try:
        out = subprocess.run([_hipcc(), "--version"], capture_output=True, text=True).stdout
    except OSError:
        out = ""
    if VALIDATED_COMPILER in out or os.environ.get("TRIFAST_ASM_MFMA") == "1":
        return []
    print(f"trifast_amd.build: hipcc is not {VALIDATED_COMPILER}: building the row-resident backward with "
          "compiler-placed MFMAs (-DTRI_MFMA_ACC_BUILTIN); set TRIFAST_ASM_MFMA=1 to keep the asm form and "
          "run the GPU tests of the row-resident kernel before trusting it", file=sys.stderr)
    return ["-DTRI_MFMA_ACC_BUILTIN"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the ROCm toolchain is required to build trifast_amd")
    return exe


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, obj: Path, verbose: bool, extra: tuple[str, ...] = ()) -> None:
    cmd = [_hipcc(), *HIPCC_FLAGS, *PER_SOURCE_FLAGS.get(src.name, []), *extra, "-I", str(CSRC), "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src.name}:\n{res.stdout}\n{res.stderr}")
    if verbose:
        # the host pass does not know the packed-fp32 feature name; that warning is noise
        noise = "packed-fp32-ops"
        msg = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
        if msg.strip():
            print(msg, file=sys.stderr)


def build(verbose: bool = False, jobs: int | None = None, out: Path | None = None, extra: tuple[str, ...] = ()) -> Path:
    """Compile every translation unit and link the shared library.  Always rebuilds.

    ``out`` writes the library elsewhere and ``extra`` appends hipcc flags (e.g. ``-DNAME``);
    the in-tree library is then left alone."""
    out = Path(out) if out else LIB_PATH
    build_dir = PKG_DIR / "build" / (out.stem if out != LIB_PATH else "main")
    build_dir.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    extra = (*extra, *_compiler_flags())
    objs = [build_dir / (s.stem + ".o") for s in srcs]
    jobs = jobs or min(len(srcs), int(os.environ.get("MAX_JOBS", "8")))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        futs = [pool.submit(_compile, s, o, verbose, tuple(extra)) for s, o in zip(srcs, objs)]
        for f in futs:
            f.result()
    tmp = out.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    print(f"built {build(verbose=True)}")
