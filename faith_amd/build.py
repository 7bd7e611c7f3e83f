"""Builds libfaith_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

    python -m faith_amd.build            # compile everything
    python -m faith_amd.build --force    # ignore time stamps

hipcc cross-compiles: no GPU is needed to build.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "obj")
LIB = os.path.join(HERE, "libfaith_amd.so")

ARCH = "gfx950"
COMMON = [
    "-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}",
    # the compiler must not form packed-fp32 instructions on its own
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]
# per-file extras
EXTRA = {
    # the relaxations round (b - x0) * k and + y0 separately, as the PyTorch path does
    "act.hip": ["-ffp-contract=off"],
    "mul.hip": ["-ffp-contract=off"],
    "affine.hip": ["-ffp-contract=off"],
    "softmax.hip": ["-ffp-contract=off"],
    # the dot product splits the intervals by sign with fmaxf / fminf: one instruction each only when the
    # compiler need not quiet signalling NaNs first
    "dot.hip": ["-fno-honor-nans"],
    "dot_tiled.hip": ["-fno-honor-nans"],
    "dot_transposed.hip": ["-fno-honor-nans"],
}


def sources():
    return sorted(f for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime():
    hs = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".h")]
    hs.append(os.path.join(os.path.dirname(HERE), "include", "faith_amd.h"))
    return max(os.path.getmtime(h) for h in hs)


def _compile(src, force):
    obj = os.path.join(OBJ, src.replace(".hip", ".o"))
    path = os.path.join(CSRC, src)
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) > max(os.path.getmtime(path), _headers_mtime())):
        return obj, False
    cmd = ["hipcc", *COMMON, *EXTRA.get(src, []), "-c", path, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    return obj, True


def build(force: bool = False, verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sources()
    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), srcs))
    objs = [o for o, _ in results]
    if force or any(c for _, c in results) or not os.path.exists(LIB):
        cmd = ["hipcc", "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", LIB]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB} from {len(srcs)} sources")
    return LIB


VARIANTS = os.path.join(HERE, "variants")
# GEMM kernel variants built ahead of time for the generate-and-recompile tuner (faith_amd.autotune): tile shapes
# the library does not ship -- (MFMA blocks per wavefront along M, along N, wavefronts per SIMD, raised priority) --
# so that a tuning run on a machine without a compiler, or one that must not compile, still has generated variants
# to measure; the tuner compiles any other point of its space on demand.
PREBUILT_VARIANTS = [(4, 1, 2, 0), (1, 4, 2, 0), (3, 1, 2, 0), (1, 3, 2, 1), (2, 2, 2, 0), (2, 1, 3, 0), (1, 2, 3, 1), (1, 1, 4, 1)]


def build_variants(verbose: bool = True):
    """Compiles PREBUILT_VARIANTS into faith_amd/variants/ (existing builds of the same source are kept)."""
    from .autotune import GemmVariantSpec, compile_gemm_variant
    with ThreadPoolExecutor(max_workers=8) as ex:
        paths = list(ex.map(lambda v: compile_gemm_variant(GemmVariantSpec(*v), VARIANTS), PREBUILT_VARIANTS))
    for name in os.listdir(VARIANTS):                      # builds of an earlier state of the sources
        if os.path.join(VARIANTS, name) not in paths:
            os.remove(os.path.join(VARIANTS, name))
    if verbose:
        print(f"built {len(paths)} GEMM variants in {VARIANTS}")
    return paths


if __name__ == "__main__":
    build(force="--force" in sys.argv)
    build_variants()
