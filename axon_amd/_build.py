"""Build recipe for libaxon_amd.so (HIP, gfx950 only).

``build()`` always recompiles; ``ensure_built()`` compiles only when the
library is missing.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import tempfile

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "libaxon_amd.so")
SOURCES = ("capi.hip", "rows.hip", "loss.hip", "owned.hip", "diag.hip", "returns.hip", "cov.hip", "logits.hip", "lmhead.hip")

HIPCC_FLAGS = (
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-munsafe-fp-atomics",  # native global_atomic_add_f32 instead of a CAS loop
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
)


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libaxon_amd.so cannot be built")
    return exe


def _run(cmd, cwd) -> str:
    proc = subprocess.run(cmd, cwd=cwd, capture_output=True, text=True)
    log = "\n".join(
        line for line in (proc.stdout + proc.stderr).splitlines()
        if "is not a recognized feature" not in line  # host pass does not know the GPU feature
    )
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{log}")
    return log


def build(verbose: bool = False) -> str:
    """Compile every HIP source into ``axon_amd/libaxon_amd.so`` and return its path.  One hipcc per source,
    side by side (the file with the most kernel instantiations takes a minute alone), then one link."""
    from concurrent.futures import ThreadPoolExecutor

    hipcc = _hipcc()
    compile_flags = [f for f in HIPCC_FLAGS if f != "-shared"]
    with tempfile.TemporaryDirectory(prefix="axon_amd_build_") as tmp:
        objs = [os.path.join(tmp, os.path.splitext(s)[0] + ".o") for s in SOURCES]
        cmds = [[hipcc, *compile_flags, "-c", os.path.join(CSRC, s), "-o", o] for s, o in zip(SOURCES, objs)]
        with ThreadPoolExecutor(max_workers=min(len(cmds), os.cpu_count() or 1, 8)) as pool:
            logs = list(pool.map(lambda c: _run(c, tmp), cmds))
        out = os.path.join(tmp, "libaxon_amd.so")
        logs.append(_run([hipcc, "--offload-arch=gfx950", "-fPIC", "-shared", "-o", out, *objs], tmp))
        if verbose and any(l.strip() for l in logs):
            print("\n".join(l for l in logs if l.strip()))
        shutil.move(out, LIB_PATH)
    return LIB_PATH


def ensure_built() -> str:
    if not os.path.exists(LIB_PATH):
        build()
    return LIB_PATH
