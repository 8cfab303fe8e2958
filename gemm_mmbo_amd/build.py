"""Build libmmbo_gemm.so (the C-ABI library with every gfx950 kernel) in-tree with hipcc.

    python -m gemm_mmbo_amd.build [--force]

Each (element type, tile row) pair is its own translation unit so the kernels compile in
parallel; objects go to gemm_mmbo_amd/csrc/build/, the library to gemm_mmbo_amd/csrc/.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB = os.path.join(CSRC, "libmmbo_gemm.so")

NUM_TILES = 6  # keep in step with csrc/configs.hpp
NUM_RING_TILES = 4
NUM_F64_TILES = 6
NUM_X16_TILES = 8

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # no packed-fp32 VALU forms: some of them have produced wrong results on this hardware
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# The direct-to-LDS kernels rely on facts about the generated code that the compiler does not guarantee: their inline
# assembly changes M0 and the accumulation registers without declaring it, and LDS reads stay in flight across
# compiler-scheduled instructions.  tests/test_kernel_asm.py checks those facts on the assembly a given hipcc generates;
# this is the compiler build it last passed with.  Another compiler may still be fine -- run that test file with it
# first (then update this string); MMBO_STRICT_TOOLCHAIN=1 turns the warning below into an error.
ASM_CHECKED_WITH = "roc-7.2.0 26014"


def _hipcc_version():
    try:
        return subprocess.run([HIPCC, "--version"], capture_output=True, text=True).stdout
    except OSError as e:
        raise RuntimeError(f"cannot run {HIPCC}: {e}")


def _check_toolchain(verbose=True):
    text = _hipcc_version()
    if ASM_CHECKED_WITH in text:
        return True
    first = (text.strip().split("\n") or ["?"])[0:2]
    msg = (f"gemm_mmbo_amd.build: {HIPCC} is not the compiler build the kernels' assembly checks passed with "
           f"(want '{ASM_CHECKED_WITH}', have: {' / '.join(first)}).  Run `python -m pytest tests/test_kernel_asm.py` with this "
           "compiler before trusting the library.")
    if os.environ.get("MMBO_STRICT_TOOLCHAIN") == "1":
        raise RuntimeError(msg)
    if verbose:
        print("WARNING: " + msg, file=sys.stderr)
    return False


def _units():
    units = [("mmbo_gemm.hip", "mmbo_gemm.o", []), ("probe.hip", "probe.o", [])]
    for dtype in (0, 1):
        for tile in range(NUM_TILES):
            units.append(("inst_staged.hip", f"inst_staged_{dtype}_{tile}.o",
                          [f"-DMMBO_DTYPE={dtype}", f"-DMMBO_TILE={tile}"]))
        for tile in range(NUM_RING_TILES):
            units.append(("inst_ring.hip", f"inst_ring_{dtype}_{tile}.o",
                          [f"-DMMBO_DTYPE={dtype}", f"-DMMBO_TILE={tile}"]))
    for dtype in (0, 1):
        for tile in range(NUM_X16_TILES):
            units.append(("inst_x16.hip", f"inst_x16_{dtype}_{tile}.o", [f"-DMMBO_DTYPE={dtype}", f"-DMMBO_TILE={tile}"]))
    for tile in range(NUM_F64_TILES):
        units.append(("inst_dgemm.hip", f"inst_dgemm_{tile}.o", [f"-DMMBO_TILE={tile}"]))
    return units


def _deps(src, seen=None):
    """The files a source depends on: itself and, recursively, everything it includes with #include "..."."""
    import re
    seen = seen if seen is not None else set()
    path = os.path.normpath(src)
    if path in seen or not os.path.exists(path):
        return seen
    seen.add(path)
    for inc in re.findall(r'^\s*#\s*include\s+"([^"]+)"', open(path).read(), flags=re.M):
        _deps(os.path.join(os.path.dirname(path), inc), seen)
    return seen


def _compile(unit, force, newest_dep):
    src, obj, defs = unit
    objp = os.path.join(OBJ, obj)
    newest_dep = max([newest_dep] + [os.path.getmtime(p) for p in _deps(os.path.join(CSRC, src))])
    if not force and os.path.exists(objp) and os.path.getmtime(objp) >= newest_dep:
        return obj, "up to date"
    cmd = [HIPCC] + FLAGS + defs + ["-c", os.path.join(CSRC, src), "-o", objp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {obj}:\n{' '.join(cmd)}\n{r.stderr[-4000:]}")
    return obj, "compiled"


def build(force=False, verbose=True, jobs=None):
    os.makedirs(OBJ, exist_ok=True)
    _check_toolchain(verbose)
    newest = os.path.getmtime(os.path.abspath(__file__))
    units = _units()
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda u: _compile(u, force, newest), units))
    if verbose:
        for obj, what in results:
            print(f"  {obj}: {what}")
    objs = [os.path.join(OBJ, u[1]) for u in units]
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stderr[-4000:]}")
    # a translation unit whose kernels silently failed to instantiate leaves the library with undefined symbols
    import ctypes
    try:
        ctypes.CDLL(LIB, mode=getattr(os, "RTLD_NOW", 2))
    except OSError as e:
        raise RuntimeError(f"{LIB} does not load: {e}")
    if verbose:
        print(f"  linked {LIB}")
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv)
