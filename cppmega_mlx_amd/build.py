"""Build recipe for libcppmega_mi355.so (hipcc, gfx950 only).

``python -m cppmega_mlx_amd.build`` compiles every ``csrc/*.hip`` translation
unit and links the shared library next to this package, where the loader in
``_lib.py`` looks for it.  hipcc cross-compiles without a GPU.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "libcppmega_mi355.so"
LIB_PATH = PKG_DIR / LIB_NAME
OBJ_DIR = PKG_DIR / "csrc" / "build"

OFFLOAD_ARCH = "gfx950"
# packed-fp32 VALU forms are kept out of the generated code on purpose.
HIPCC_FLAGS = [
    f"--offload-arch={OFFLOAD_ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA builtins keep their accumulators in ordinary VGPRs; kernels that want AGPR
    # accumulators say so with inline assembly
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
    "-Wno-unused-result",
]

# Per-file additions (none at present).
FILE_FLAGS: dict[str, list[str]] = {}
# Kernels (mangled-name fragments) that must not use scratch memory: they wait for their
# asynchronous loads by count, and spill traffic would be counted with them.
NO_SCRATCH = {
    "sparse_mla_latent.hip": ("sparse_mla_latent_kernel",),
}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc, PATH)")


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _compile_one(hipcc: str, src: Path, verbose: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [hipcc, *HIPCC_FLAGS, *FILE_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
    if src.name in NO_SCRATCH:
        cmd.append("-Rpass-analysis=kernel-resource-usage")
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{proc.stdout}\n{proc.stderr}")
    if src.name in NO_SCRATCH:
        _check_no_scratch(src.name, proc.stderr)
    errs = [ln for ln in proc.stderr.splitlines()
            if "packed-fp32-ops" not in ln and "kernel-resource-usage" not in ln and ln.strip()]
    if verbose and errs:
        print("\n".join(errs), flush=True)
    return obj


def _check_no_scratch(name: str, remarks: str) -> None:
    """Parse the compiler's resource remarks: fail the build if a listed kernel spills."""
    current = None
    for ln in remarks.splitlines():
        if "Function Name:" in ln:
            current = ln.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in ln and current:
            size = int(ln.split("ScratchSize [bytes/lane]:")[1].split("[")[0].strip())
            if size and any(frag in current for frag in NO_SCRATCH[name]):
                raise RuntimeError(f"{name}: kernel {current} uses {size} bytes/lane of scratch memory; "
                                   "it must fit its registers (see NO_SCRATCH in build.py)")


def build(verbose: bool = True, jobs: int | None = None) -> Path:
    """Compile all kernels for gfx950 and link the shared library. Always rebuilds."""
    hipcc = _hipcc()
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(len(srcs), 8)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile_one(hipcc, s, verbose), srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc, f"--offload-arch={OFFLOAD_ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stdout}\n{proc.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build(verbose="-q" not in sys.argv)
    print(f"built {path}")
