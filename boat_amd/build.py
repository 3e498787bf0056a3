"""Build libboat_amd.so for gfx950: HIP kernels (hipcc) + the C host side (gcc), one shared library.

    python -m boat_amd.build            # compile everything into boat_amd/lib/libboat_amd.so

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere ROCm is installed.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "boat_amd" / "csrc"
OBJ = ROOT / "boat_amd" / "lib" / "obj"
LIB = ROOT / "boat_amd" / "lib" / "libboat_amd.so"
ROCM = Path(os.environ.get("ROCM_PATH", "/opt/rocm"))
HIPCC = str(ROCM / "bin" / "hipcc")

HIP_SOURCES = sorted((CSRC / "hip").glob("*.hip"))
C_SOURCES = sorted((CSRC / "host").glob("*.c"))
EXAMPLES = sorted((ROOT / "boat_amd" / "examples").glob("*.c"))   # C programs against include/boat_api.h

# -ffp-contract=off: a*b+c stays two roundings, like the reference's scalar C loops.
# packed-fp32 ops are switched off for every device compile.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    f"-I{ROOT / 'include'}", f"-I{CSRC / 'hip'}",
]
C_FLAGS = [
    "-O2", "-std=c11", "-fPIC", "-ffp-contract=off", "-Wall", "-Wextra", "-fvisibility=hidden", "-D_GNU_SOURCE",
    f"-I{ROOT / 'include'}", f"-I{CSRC / 'host'}",
]


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{proc.stdout}\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")


def _compile_hip(src: Path) -> Path:
    """Compile one HIP source and refuse kernels that spill registers to scratch memory: a dispatch that needs scratch
    makes the runtime set it up for the queue, and on MI355X every later launch of the process then takes several
    microseconds longer (measured on the small-GEMM kernels: 7 us against 4 us)."""
    out = OBJ / (src.stem + ".o")
    proc = subprocess.run([HIPCC, *HIP_FLAGS, "-Rpass-analysis=kernel-resource-usage", "-fno-caret-diagnostics", "-c", str(src), "-o", str(out)],
                          capture_output=True, text=True)
    if proc.returncode != 0:
        noise = "is not a recognized feature for this target"
        err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l and "-Rpass-analysis" not in l)
        raise RuntimeError(f"hipcc failed ({proc.returncode}) on {src}\n{proc.stdout}\n{err}")
    kernel, spilling = None, []
    for line in proc.stderr.splitlines():
        if "Function Name:" in line:
            kernel = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            if int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0]) > 0:
                spilling.append(kernel)
    if spilling:
        raise RuntimeError(f"{src.name}: kernels that need scratch memory (register spills): {spilling}")
    warnings = [l for l in proc.stderr.splitlines()
                if "-Rpass-analysis" not in l and "is not a recognized feature for this target" not in l
                and not l.startswith("In file included from") and l.strip()]
    if warnings:
        sys.stderr.write("\n".join(warnings) + "\n")
    return out


def _compile_c(src: Path) -> Path:
    out = OBJ / (src.stem + ".o")
    _run(["gcc", *C_FLAGS, "-c", str(src), "-o", str(out)])
    return out


def build_all(jobs: int = 8, verbose: bool = True) -> Path:
    """Compile every source and link boat_amd/lib/libboat_amd.so; returns its path."""
    OBJ.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        hip_objs = list(pool.map(_compile_hip, HIP_SOURCES))
        c_objs = list(pool.map(_compile_c, C_SOURCES))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB),
          *map(str, hip_objs), *map(str, c_objs), "-lm", f"-Wl,-rpath,{ROCM / 'lib'}"])
    for src in EXAMPLES:   # linked against the library exactly as a Boat program would be re-linked
        _run(["gcc", "-O2", "-std=c11", "-D_GNU_SOURCE", f"-I{ROOT / 'include'}", str(src), "-o", str(LIB.parent / src.stem),
              f"-L{LIB.parent}", "-lboat_amd", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath-link,{ROCM / 'lib'}", "-lm"])
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size // 1024} KiB) from {len(hip_objs)} HIP + {len(c_objs)} C sources, "
              f"{len(EXAMPLES)} example program(s)")
    return LIB


if __name__ == "__main__":
    build_all()
