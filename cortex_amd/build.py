"""Builds libcortex_hip.so for gfx950 with hipcc.

Every translation unit under ``csrc/`` is compiled to an object file in
parallel and linked into ``cortex_amd/libcortex_hip.so``.  The library is kept
in-tree (it is ignored by git) so that a run on another machine can load it
without building.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
LIB = HERE / "libcortex_hip.so"

SOURCES = [
    "plan.cpp",
    "elementwise.cpp",
    "driver.hip",
    "ops_assign.hip",
    "ops_unary.hip",
    "ops_binary.hip",
    "ops_binary_f32.hip",
    "ops_binary_f64.hip",
    "ops_binary_int_narrow.hip",
    "ops_binary_int_wide.hip",
    "ops_ternary.hip",
    "ops_accum.hip",
    "ops_accum_stream.hip",
    "ops_reduce.hip",
    "ops_reduce_int.hip",
    "ops_reduce_int_b.hip",
    "ops_reduce_int_c.hip",
    "ops_optim.hip",
    "ops_nn.hip",
    "ops_batchnorm.hip",
    "ops_rand.hip",
    "ops_blas.cpp",
    "ops_gemv.hip", "ops_pool.hip", "ops_conv.hip", "ops_lrn.hip",
]

# -ffp-contract=off: the reference's CPU backend rounds after every JVM
# operation, so no multiply-add may be fused behind the functors' backs.
# The packed-fp32 feature is switched off for the device pass.
# --offload-compress: the device code of every object is stored compressed and
# unpacked by the HIP runtime when the library is loaded (about a quarter of the size).
FLAGS = [
    "-O3",
    "--offload-arch=gfx950",
    "-fPIC",
    "-std=c++17",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "--offload-compress",
    "-Wno-unused-command-line-argument",
    "-Wall",
]


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _dependencies(depfile: Path):
    """The files a make-style dependency file names, or None when it cannot be read."""
    try:
        text = depfile.read_text().replace("\\\n", " ")
    except OSError:
        return None
    deps = []
    for rule in text.splitlines():
        _, sep, rest = rule.partition(":")
        if sep:
            deps.extend(Path(d) for d in rest.split())
    return deps


def _compile(src: str, force: bool) -> Path:
    """Compiles one source; without `force`, only when it or a header it includes (as recorded by the compiler
    in the object's dependency file at the last build) is newer than the object."""
    obj = CSRC / "build" / (Path(src).stem + ".o")
    depfile = obj.with_suffix(".d")
    obj.parent.mkdir(exist_ok=True)
    path = CSRC / src
    if not force and obj.exists():
        deps = _dependencies(depfile)
        if deps is None:
            deps = [path] + list(CSRC.glob("*.h")) + [HERE.parent / "include" / "cortex_hip.h"]
        own = [d for d in deps + [path] if CSRC in d.resolve().parents or d.resolve().parent == (HERE.parent / "include")]
        if all(d.exists() and obj.stat().st_mtime >= d.stat().st_mtime for d in own):
            return obj
    cmd = [_hipcc(), *FLAGS, "-MD", "-MF", str(depfile), "-x", "hip", "-c", str(path), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, jobs: int | None = None) -> Path:
    """Compiles every source and links the shared library; returns its path."""
    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force), SOURCES))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB


if __name__ == "__main__":
    print(build(force="--incremental" not in sys.argv))
