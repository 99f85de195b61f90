"""Builds libmonet_hip.so (the gfx950 kernels) in-tree with hipcc.

`python -m monet_amd.build` compiles every `csrc/*.hip` for gfx950 and links
`monet_amd/libmonet_hip.so`.  No GPU is needed to build.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libmonet_hip.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"
# packed-fp32 instruction selection is switched off for every device object
FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(CSRC.glob("*.hip"))


def _compile(src: Path, obj: Path):
    cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stdout}\n{r.stderr}")
    return r.stderr


def build_library(verbose: bool = True, jobs: int = 8) -> Path:
    """Compile all kernels (always recompiles) and link the shared library."""
    objdir = PKG_DIR / "build"
    objdir.mkdir(exist_ok=True)
    srcs = sources()
    objs = [objdir / (s.stem + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for s, warn in zip(srcs, ex.map(_compile, srcs, objs)):
            if verbose:
                kept = [l for l in warn.splitlines() if "packed-fp32-ops" not in l and l.strip()]
                print(f"[monet_amd.build] {s.name} ok" + (("\n" + "\n".join(kept)) if kept else ""))
    cmd = [HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"[monet_amd.build] linked {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    sys.exit(0)
