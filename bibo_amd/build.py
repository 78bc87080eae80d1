"""Build recipe for libbibo_moe.so: every .hip file under csrc/ compiled for gfx950 with hipcc and
linked into one shared library next to this file.  `python -m bibo_amd.build` runs it."""
from __future__ import annotations

import os
import pathlib
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = pathlib.Path(__file__).resolve().parent
CSRC = HERE / "csrc"
BUILD = HERE / "csrc" / "build"
LIB = HERE / "libbibo_moe.so"

SOURCES = ["router.hip", "permute.hip", "experts_generic.hip", "experts_mfma.hip", "experts_fused.hip", "experts_stream.hip", "ffn.hip", "backward.hip", "backward_generic.hip", "api.hip"]

# -packed-fp32-ops is switched off on purpose: hipcc -O3 otherwise forms v_pk_*_f32 from scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: the HIP extension cannot be built on this machine")
    return exe


def _compile(src: str, extra: list[str]) -> pathlib.Path:
    obj = BUILD / (src + ".o")
    cmd = [hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
    if r.stderr.strip():
        # the host pass warns that it does not know -packed-fp32-ops; that is harmless
        lines = [l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l and l.strip()]
        if lines:
            sys.stderr.write("\n".join(lines) + "\n")
    return obj


def build(extra_flags: list[str] | None = None, jobs: int = 4) -> pathlib.Path:
    """Compile every source and link the shared library; always recompiles."""
    BUILD.mkdir(parents=True, exist_ok=True)
    extra = list(extra_flags or [])
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), SOURCES))
    tmp = LIB.with_suffix(".so.tmp")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build(sys.argv[1:]))
