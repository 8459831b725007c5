"""Builds the native half of hc_amd in-tree.

    python -m hc_amd.build            # everything
    python -m hc_amd.build gemm       # one kernel module, then relink
    python -m hc_amd.build --probes   # everything, with the measurement builds
                                      # of the GEMM (kernels whose output is not
                                      # the product; hc_amd_bench.h), which a
                                      # default build leaves out

Outputs (all under hc_amd/_native/, none tracked by git):
    build/<module>.hsaco      gfx950 code objects, one per kernels/<module>.hip
    libhc_amd_runtime.so      C ABI (ol*, hcgpu*, hcamd*) with the code objects
                              embedded in its read-only data
    libhc_amd_pyabi.so        PyObject* conversions (needs CPython headers)

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm
toolchain is installed.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
NATIVE = PKG / "_native"
BUILD = NATIVE / "build"
INCLUDE = PKG.parent / "include"

KERNEL_MODULES = ("copy", "elementwise", "map", "imap", "fmap", "distance", "gather", "softmax", "quantize", "gemm")
ARCH = "gfx950"

# Packed fp32 VALU forms are kept out of every kernel.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# The map kernel is an interpreter whose branches are all wave-uniform; left
# alone, the compiler linearises them into a chain of guarded regions with
# register copies at every join.
MODULE_FLAGS = {"map": ["-mllvm", "--structurizecfg-skip-uniform-regions"]}


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the ROCm toolchain is required")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature and says so on
    # every invocation; that line carries no information.
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed: {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        print(err, file=sys.stderr)


PROBES = False          # set by --probes: compile the measurement builds too


def _defines() -> list[str]:
    return ["-DHCAMD_PROBES"] if PROBES else []


def build_kernel_module(name: str, keep_asm: bool = False) -> Path:
    src = CSRC / "kernels" / f"{name}.hip"
    out = BUILD / f"{name}.hsaco"
    cmd = [_hipcc(), "--genco", "--no-gpu-bundle-output", *DEVICE_FLAGS, *_defines(),
           *MODULE_FLAGS.get(name, []), "-I", str(CSRC / "kernels"),
           "-o", str(out), str(src)]
    if keep_asm:
        cmd.insert(2, "-save-temps=obj")
    _run(cmd)
    return out


def _rocm_root() -> Path:
    return Path(os.environ.get("ROCM_PATH") or Path(_hipcc()).resolve().parents[1])


def build_scratch() -> Path:
    # The one source with both host and device code: the static device scratch
    # array of the entry point that allocates nothing has to be a registered
    # device symbol, so hipcc compiles it into an ordinary object.
    out = BUILD / "scratch.o"
    _run([_hipcc(), "-c", "-fPIC", *DEVICE_FLAGS, "-I", str(INCLUDE), "-I", str(CSRC),
          "-o", str(out), str(CSRC / "scratch.hip")])
    return out


def build_runtime() -> Path:
    # Host-only C++ on the HIP runtime API: the host compiler builds it and
    # links libamdhip64; blobs.S pulls the code objects in with .incbin.
    out = NATIVE / "libhc_amd_runtime.so"
    rocm = _rocm_root()
    cxx = shutil.which("g++") or "g++"
    scratch = build_scratch()
    _run([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", *_defines(),
          "-D__HIP_PLATFORM_AMD__", "-I", str(rocm / "include"),
          "-I", str(INCLUDE), "-I", str(CSRC), f"-Wa,-I{BUILD}",
          str(CSRC / "runtime.cpp"), str(CSRC / "blobs.S"), str(scratch),
          "-o", str(out),
          f"-L{rocm / 'lib'}", f"-Wl,-rpath,{rocm / 'lib'}", "-lamdhip64"])
    return out


def build_pyabi() -> Path:
    out = NATIVE / "libhc_amd_pyabi.so"
    cxx = shutil.which("g++") or "g++"
    _run([cxx, "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
          "-I", sysconfig.get_paths()["include"], "-I", str(INCLUDE),
          str(CSRC / "pyabi.cpp"), "-o", str(out), "-ldl"])
    return out


def build_all(modules: tuple[str, ...] = KERNEL_MODULES, keep_asm: bool = False) -> None:
    BUILD.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(modules) or 1)) as pool:
        list(pool.map(lambda m: build_kernel_module(m, keep_asm), modules))
    missing = [m for m in KERNEL_MODULES if not (BUILD / f"{m}.hsaco").exists()]
    if missing:
        raise RuntimeError(f"code objects missing, build them first: {missing}")
    build_runtime()
    build_pyabi()


def main(argv: list[str]) -> int:
    global PROBES
    keep = "--asm" in argv
    PROBES = "--probes" in argv
    names = tuple(a for a in argv if not a.startswith("--")) or KERNEL_MODULES
    unknown = [n for n in names if n not in KERNEL_MODULES]
    if unknown:
        print(f"unknown kernel module(s): {unknown}; known: {KERNEL_MODULES}",
              file=sys.stderr)
        return 2
    build_all(names, keep)
    print(f"built {', '.join(names)} -> {NATIVE}")
    return 0


if __name__ == "__main__":
    sys.exit(main(sys.argv[1:]))
