"""Build recipe of the native library (HIP kernels + C ABI + C++ host layer).

    python scpaper-2021_amd/build.py            # compile everything for gfx950

hipcc cross-compiles for gfx950 without a GPU.  Objects go to
``scpaper-2021_amd/build/`` and the shared library to
``scpaper-2021_amd/lib/libet_hip.so`` (both ignored by git; the library
travels with the source tree to the GPU machine).
"""
from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
ROOT = PKG.parent
BUILD = PKG / "build"
LIBDIR = PKG / "lib"
LIB = LIBDIR / "libet_hip.so"

ARCH = "gfx950"
HIPCC = os.environ.get("HIPCC") or shutil.which("hipcc") or "/opt/rocm/bin/hipcc"

COMMON = ["-O3", "-std=c++17", "-fPIC", "-I", str(ROOT / "include"), "-Wall", "-Wno-unused-function"]
# Packed-fp32 code generation is switched off for device code.
DEVICE = [f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
          "-Wno-unknown-warning-option", "-Wno-unused-command-line-argument",
          "-Rpass-analysis=kernel-resource-usage"]  # registers and scratch of every kernel, kept in RESOURCES
RESOURCES = LIBDIR / "kernel_resources.txt"
_resource_lines: list[str] = []


def sources() -> list[Path]:
    return sorted((PKG / "csrc").glob("*.hip")) + sorted((PKG / "host").glob("*.cpp"))


def _compile(src: Path) -> Path:
    obj = BUILD / (src.name + ".o")
    cmd = [HIPCC, *COMMON]
    if src.suffix == ".hip":
        cmd += DEVICE
    else:
        cmd += ["-x", "c++"]  # host-only translation unit: no device pass
    cmd += ["-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass does not know the packed-fp32 feature name; that
    # warning is expected and dropped here.
    noise = ("is not a recognized feature for this target", "'-packed-fp32-ops'")
    lines = [l for l in res.stderr.splitlines() if not any(n in l for n in noise)]
    # "file:line:col: remark: Function Name: f [-Rpass-analysis=...]", then "remark:     VGPRs: n [...]" lines,
    # each followed by two lines of source context
    name = None
    kept = []
    skip_context = 0
    for l in lines:
        if "remark:" in l and "[-Rpass-analysis=kernel-resource-usage]" in l:
            text = l.split("remark:", 1)[1].replace("[-Rpass-analysis=kernel-resource-usage]", "").strip()
            if text.startswith("Function Name:"):
                name = text.split(":", 1)[1].strip()
                _resource_lines.append(f"{src.name} {name}")
            elif name and text.split(":")[0] in ("TotalSGPRs", "VGPRs", "AGPRs", "ScratchSize [bytes/lane]", "Occupancy [waves/SIMD]",
                                                  "SGPRs Spill", "VGPRs Spill", "LDS Size [bytes/block]"):
                _resource_lines[-1] += " | " + text
            skip_context = 2
            continue
        if skip_context and ("|" in l):
            skip_context -= 1
            continue
        skip_context = 0
        kept.append(l)
    err = "\n".join(kept)
    if res.returncode != 0:
        raise RuntimeError(f"compile failed: {' '.join(cmd)}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_all(jobs: int | None = None, verbose: bool = True) -> Path:
    """Compile every source for gfx950 and link the shared library."""
    BUILD.mkdir(exist_ok=True)
    LIBDIR.mkdir(exist_ok=True)
    _resource_lines.clear()
    srcs = sources()
    jobs = jobs or min(8, len(srcs))
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    tmp = LIB.with_suffix(".so.tmp")
    cmd = [HIPCC, "-shared", "-fPIC", f"--offload-arch={ARCH}", *map(str, objs), "-lz", "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed: {' '.join(cmd)}\n{res.stderr}")
    os.replace(tmp, LIB)
    RESOURCES.write_text("\n".join(sorted(_resource_lines)) + "\n")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    build_programs(verbose)
    return LIB


# C++ programs written against the class layer (include/et/*.h) and linked with the library.
PROGRAMS = {ROOT / "tests" / "cpp" / "class_layer_cases.cpp": ROOT / "tests" / "cpp" / "bin" / "class_layer_cases",
            PKG / "programs" / "et_sweeps.cpp": PKG / "bin" / "et_sweeps"}


def build_programs(verbose: bool = True) -> None:
    for src, exe in PROGRAMS.items():
        if not src.exists():
            continue
        exe.parent.mkdir(exist_ok=True)
        rel = os.path.relpath(LIBDIR, exe.parent)  # the tree may be copied elsewhere: rpath relative to the program
        cmd = [HIPCC, *COMMON, "-x", "c++", str(src), "-L", str(LIBDIR), "-let_hip",
               f"-Wl,-rpath,{LIBDIR}", f"-Wl,-rpath,$ORIGIN/{rel}", "-o", str(exe)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"program build failed: {' '.join(cmd)}\n{res.stderr}")
        if verbose:
            print(f"built {exe}")


if __name__ == "__main__":
    build_all()
